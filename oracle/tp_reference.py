"""CPU restatement of the reference's tensor-parallel hot path.  TEST INFRASTRUCTURE ONLY.

Nothing under ``merak_amd/`` imports this module: it exists to check the HIP
kernels (``tests/``, ``__graft_entry__.smoke()``) and to be timed as the CPU
baseline (``bench.py``).  It is written fresh from a reading of the reference,
in the reference's op order, with plain torch CPU ops — which is what the
reference itself executes (it has no kernels of its own; every FLOP is
``F.linear`` / ``F.embedding`` / ``torch.max/exp/sum/log`` / ``torch.argmax``).
Each function cites the reference lines it follows.

How each function is pinned (tests/test_oracle_pins.py); the reference's own
tests hold no golden vectors or numeric assertions for this path, so the pins
are closed forms, library routines and brute force:

  column/row forward      F.linear *is* the reference op; brute-force triple loop; fp64 matmul
  linear_backward         torch.autograd.grad of the fp64 forward; gradcheck
  gelu_new / swiglu       math.tanh / math.exp scalar loops; autograd for the derivatives
  embedding forward       table[ids] exact; shard rows out of range are exactly zero
  embedding_backward      autograd of F.embedding; brute-force loop
  cross entropy forward   F.cross_entropy(reduction='none') in range;
                          logsumexp(x) - max(x) for out-of-range targets (-100 included)
  cross entropy backward  autograd.grad of the fp64 closed-form loss
  partials + combine      8 vocab slices combined == full-vocab result
  shard_master_weight     hand-written table for stride 1 and 2 (tests/golden/shard_table.json)
  greedy_argmax           brute-force scan, first index on ties
  VocabUtility / divide   integer closed forms
  top_k_logits            hand-worked cases (k-th value ties, the token that crosses top_p stays, first token
                          always stays); transformers' TopKLogitsWarper / TopPLogitsWarper on random logits
  sample_tail             numpy.searchsorted on the cumulative distribution; draw frequencies over 40000
                          uniforms against the probabilities (torch.multinomial's own random stream cannot be
                          reproduced, so the draw takes the uniforms as an argument)
  decode_step             reduces to the plain linears, swiglu and greedy_argmax above on the same inputs
  rms_norm                transformers' LlamaRMSNorm module; constant rows (closed form 3 / sqrt(9 + eps))
  rope_tables, apply_rope transformers' LlamaRotaryEmbedding + apply_rotary_pos_emb; position 0 is the identity
    (rotate_half)
  attn_decode             torch's scaled_dot_product_attention over the valid prefix with the kv heads repeated
                          per group; a single cached token returns its value; entries past the valid length
                          (junk, NaN) do not change the result
  llama_block_step        token by token through the cache == the full-sequence forward of a random-weight
                          transformers LlamaForCausalLM (the row the reference slices out of it)

The third-party arithmetic under all of this is PyTorch (the reference pins
torch>=2.0.0, setup.py:46) and, for the activations, transformers
(>4.20.0,<=4.47.0, setup.py:48): gelu_new and LlamaMLP's silu(gate)*up are
restated here from their published formulas.
"""
from __future__ import annotations

import math
from typing import Optional, Tuple

import torch
import torch.nn.functional as F


# --------------------------------------------------------------------------- integer helpers
def ensure_divisibility(numerator, denominator):
    """Merak/core/mpu/utils.py:33-36."""
    assert numerator % denominator == 0, '{} is not divisible by {}'.format(numerator, denominator)


def divide(numerator, denominator):
    """Merak/core/mpu/utils.py:39-43."""
    ensure_divisibility(numerator, denominator)
    return numerator // denominator


def vocab_range_from_per_partition_vocab_size(per_partition_vocab_size, rank, world_size):
    """Merak/core/mpu/utils.py:95-100."""
    index_f = rank * per_partition_vocab_size
    return index_f, index_f + per_partition_vocab_size


def vocab_range_from_global_vocab_size(global_vocab_size, rank, world_size):
    """Merak/core/mpu/utils.py:102-106."""
    return vocab_range_from_per_partition_vocab_size(divide(global_vocab_size, world_size), rank, world_size)


def shard_master_weight(master_weight: torch.Tensor, per_partition_size: int, partition_dim: int, stride: int,
                        rank: int, world_size: int) -> torch.Tensor:
    """This rank's shard of a full [out, in] weight: split into chunks of per_partition_size/stride along
    partition_dim, keep chunks rank, rank+world, ..., concatenate (Merak/core/mpu/layers.py:78-86)."""
    per_partition_per_stride_size = divide(per_partition_size, stride)
    weight_list = torch.split(master_weight, per_partition_per_stride_size, dim=partition_dim)
    return torch.cat(weight_list[rank::world_size], dim=partition_dim)


# --------------------------------------------------------------------------- activations (transformers)
def gelu_new(x: torch.Tensor) -> torch.Tensor:
    """HF NewGELUActivation: 0.5 x (1 + tanh(sqrt(2/pi) (x + 0.044715 x^3))) — the op between GPT-2's
    column (c_fc) and row (c_proj) linears."""
    return 0.5 * x * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (x + 0.044715 * torch.pow(x, 3.0))))


def gelu_new_grad(x: torch.Tensor) -> torch.Tensor:
    """d gelu_new / dx, closed form."""
    k0, k1 = math.sqrt(2.0 / math.pi), 0.044715
    u = k0 * (x + k1 * x ** 3)
    t = torch.tanh(u)
    return 0.5 * (1.0 + t) + 0.5 * x * (1.0 - t * t) * k0 * (1.0 + 3.0 * k1 * x * x)


def swiglu(y: torch.Tensor) -> torch.Tensor:
    """HF LlamaMLP: act_fn(gate_proj(x)) * up_proj(x) with gate and up stacked as y = [gate | up]."""
    h = y.shape[-1] // 2
    return F.silu(y[..., :h]) * y[..., h:]


def swiglu_backward(dact: torch.Tensor, y: torch.Tensor) -> torch.Tensor:
    """Gradient of swiglu w.r.t. y = [gate | up], closed form."""
    h = y.shape[-1] // 2
    gate, up = y[..., :h], y[..., h:]
    s = torch.sigmoid(gate)
    silu = gate * s
    return torch.cat([dact * up * (s + silu * (1.0 - s)), dact * silu], dim=-1)


# --------------------------------------------------------------------------- linear layers
def column_parallel_linear_forward(x, weight, bias, skip_bias_add=False):
    """ColumnParallelLinear.forward at tensor-parallel size 1 (Merak/core/mpu/layers.py:246-259):
    copy_to_model_parallel_region is the identity, bias goes into F.linear unless skip_bias_add,
    gather is the identity; returns (output, output_bias)."""
    b = bias if not skip_bias_add else None
    output = F.linear(x, weight, b)
    return output, (bias if skip_bias_add else None)


def row_parallel_linear_forward(x, weight, bias, skip_bias_add=False):
    """RowParallelLinear.forward at size 1 (layers.py:347-363): F.linear without bias, identity reduce,
    then ``output_ + bias``; returns (output, output_bias)."""
    output_ = F.linear(x, weight)
    if not skip_bias_add:
        output = output_ + bias if bias is not None else output_
        return output, None
    return output_, bias


def linear_backward(x, weight, dy, has_bias: bool):
    """What autograd derives for F.linear: dX = dY W, dW = dY^T X, db = sum over tokens of dY."""
    x2 = x.reshape(-1, x.shape[-1])
    dy2 = dy.reshape(-1, dy.shape[-1])
    dx = (dy2 @ weight).reshape(x.shape)
    dw = dy2.t() @ x2
    db = dy2.sum(0) if has_bias else None
    return dx, dw, db


# --------------------------------------------------------------------------- embedding
def vocab_parallel_embedding_forward(ids, weight, vocab_start, vocab_end, world_size):
    """VocabParallelEmbedding.forward (layers.py:145-165) for one rank's table slice."""
    if world_size > 1:
        input_mask = (ids < vocab_start) | (ids >= vocab_end)
        masked_input = ids.clone() - vocab_start
        masked_input[input_mask] = 0
    else:
        masked_input = ids
    output_parallel = F.embedding(masked_input, weight)
    if world_size > 1:
        output_parallel[input_mask, :] = 0.0
    return output_parallel  # the all-reduce over ranks (:164) is the caller's


def embedding_backward(ids, dout, rows, vocab_start, vocab_end):
    """Dense gradient of the lookup in fp32: rows of dout scatter-added at ids - start (in range only)."""
    flat = ids.reshape(-1)
    d2 = dout.reshape(-1, dout.shape[-1]).float()
    keep = (flat >= vocab_start) & (flat < vocab_end)
    dtable = torch.zeros(rows, dout.shape[-1], dtype=torch.float32)
    dtable.index_add_(0, (flat[keep] - vocab_start), d2[keep])
    return dtable


# --------------------------------------------------------------------------- cross entropy
def vocab_parallel_cross_entropy_forward(vocab_parallel_logits, target, vocab_start, vocab_end, group=None):
    """_VocabParallelCrossEntropy.forward (Merak/core/mpu/cross_entropy.py:29-83), op for op and IN PLACE on
    ``vocab_parallel_logits`` like the reference.  Returns (loss, softmax, target_mask, masked_target_1d);
    ``softmax`` aliases the input.  ``group``: a torch.distributed group to run the three all-reduces on
    (a 1-rank gloo group for the timed baseline); None skips them, which is the same thing on one rank."""
    import torch.distributed as dist
    logits_max = torch.max(vocab_parallel_logits, dim=-1)[0]                      # :32
    if group is not None:
        dist.all_reduce(logits_max, op=dist.ReduceOp.MAX, group=group)            # :33
    vocab_parallel_logits.sub_(logits_max.unsqueeze(dim=-1))                      # :37
    partition_vocab_size = vocab_parallel_logits.size()[-1]
    target_mask = (target < vocab_start) | (target >= vocab_end)                  # :48
    masked_target = target.clone() - vocab_start                                  # :49
    masked_target[target_mask] = 0                                                # :50
    logits_2d = vocab_parallel_logits.view(-1, partition_vocab_size)              # :55
    masked_target_1d = masked_target.view(-1)
    arange_1d = torch.arange(start=0, end=logits_2d.size()[0])
    predicted_logits_1d = logits_2d[arange_1d, masked_target_1d]                  # :59
    predicted_logits_1d = predicted_logits_1d.clone().contiguous()
    predicted_logits = predicted_logits_1d.view_as(target)
    predicted_logits[target_mask] = 0.0                                           # :62
    if group is not None:
        dist.all_reduce(predicted_logits, op=dist.ReduceOp.SUM, group=group)      # :64
    exp_logits = vocab_parallel_logits
    torch.exp(vocab_parallel_logits, out=exp_logits)                              # :70
    sum_exp_logits = exp_logits.sum(dim=-1)                                       # :71
    if group is not None:
        dist.all_reduce(sum_exp_logits, op=dist.ReduceOp.SUM, group=group)        # :72
    loss = torch.log(sum_exp_logits) - predicted_logits                           # :77
    exp_logits.div_(sum_exp_logits.unsqueeze(dim=-1))                             # :80
    return loss, exp_logits, target_mask, masked_target_1d


def vocab_parallel_cross_entropy_backward(softmax, target_mask, masked_target_1d, grad_output):
    """_VocabParallelCrossEntropy.backward (cross_entropy.py:86-106), in place on ``softmax``."""
    grad_input = softmax
    partition_vocab_size = softmax.size()[-1]
    grad_2d = grad_input.view(-1, partition_vocab_size)
    arange_1d = torch.arange(start=0, end=grad_2d.size()[0])
    grad_2d[arange_1d, masked_target_1d] -= (1.0 - target_mask.view(-1).float()).to(grad_2d.dtype)   # :100-101
    grad_input.mul_(grad_output.unsqueeze(dim=-1))                                                  # :104
    return grad_input


def cross_entropy_fp32(logits, target, vocab_start=0, grad_output=None):
    """The reference algorithm applied to ``logits.float()``: (loss fp32, grad fp32 or None).

    For bf16 logits the reference runs every op in bf16 (no upcast anywhere), which cannot meet a 1e-5
    loss tolerance; the oracle for bf16 inputs is therefore the same algorithm in fp32 arithmetic."""
    x = logits.detach().float().clone()
    v = x.shape[-1]
    loss, softmax, mask, mt = vocab_parallel_cross_entropy_forward(x, target, vocab_start, vocab_start + v)
    if grad_output is None:
        return loss, None
    grad = vocab_parallel_cross_entropy_backward(softmax, mask, mt, grad_output.float().reshape(target.shape))
    return loss, grad


def cross_entropy_partials(logits, target, vocab_start):
    """One rank's (row_max, row_sumexp relative to that max, raw predicted logit or 0, in-range mask) over
    its slice — the quantities behind the all-reduces of cross_entropy.py:33,64,72."""
    x = logits.float()
    v = x.shape[-1]
    m = x.max(-1).values
    s = torch.exp(x - m.unsqueeze(-1)).sum(-1)
    mask = (target < vocab_start) | (target >= vocab_start + v)
    t = (target - vocab_start).masked_fill(mask, 0)
    pred = x.gather(-1, t.unsqueeze(-1)).squeeze(-1).masked_fill(mask, 0.0)
    return m, s, pred, ~mask


def combine_partials(maxes, sums, preds, in_ranges):
    """MAX / SUM / SUM over ranks (cross_entropy.py:33,64,72) -> (loss, global_max, global_sumexp).

    The reference gathers the predicted logit after subtracting the global max, so the raw logits are
    shifted here wherever some rank owned the target."""
    gm = torch.stack(list(maxes)).max(0).values
    gs = sum(s * torch.exp(m - gm) for m, s in zip(maxes, sums))
    owned = torch.stack(list(in_ranges)).any(0)
    pred = sum(preds) - gm * owned.float()
    return torch.log(gs) - pred, gm, gs


# --------------------------------------------------------------------------- decode tail
def greedy_argmax(logits: torch.Tensor) -> torch.Tensor:
    """prev = torch.argmax(logits, dim=-1).view(-1) (Merak/inference/text_generation_inference.py:226-227)."""
    return torch.argmax(logits, dim=-1).view(-1)


def decode_step(x, w_qkv, w_gate_up, w_down, w_lm_head):
    """Single-token rows through the block's linears and the LM head, fp32 math, bf16 rounding between
    layers as a bf16 model would store them; greedy pick at the end (:223,227)."""
    def lin(a, w):
        return F.linear(a.float(), w.float())
    qkv = lin(x, w_qkv).to(x.dtype)
    y = lin(x, w_gate_up).to(x.dtype)
    h = swiglu(y.float()).to(x.dtype)
    out = lin(h, w_down).to(x.dtype)
    logits = lin(out, w_lm_head)
    return qkv, out, logits, greedy_argmax(logits)


def top_k_logits(logits, top_k=0, top_p=0.0, filter_value=-float("inf")):
    """top_k_logits of Merak/inference/text_generation_inference.py:35-69, op for op, IN PLACE on ``logits``
    ([B, V] fp32) like the reference."""
    if top_k > 0:
        kth = torch.topk(logits, top_k)[0][..., -1, None]                       # :50
        logits[logits < kth] = filter_value                                      # :50-51
    if top_p > 0.0:
        sorted_logits, sorted_indices = torch.sort(logits, descending=True, dim=-1)   # :55-56
        cumulative_probs = torch.cumsum(F.softmax(sorted_logits, dim=-1), dim=-1)     # :57-58
        remove = cumulative_probs > top_p                                        # :61
        remove[..., 1:] = remove[..., :-1].clone()                               # :64
        remove[..., 0] = 0                                                       # :65
        for i in range(sorted_indices.size(0)):                                  # :66-68
            logits[i][sorted_indices[i][remove[i]]] = filter_value
    return logits


def sample_tail(logits, temperature, top_k, top_p, uniforms):
    """The sampling branch of the generation loop (:229-235): float(), /= temperature, top_k_logits, softmax,
    one draw per row.  torch.multinomial's random stream cannot be reproduced outside torch, so the draw is
    the inverse CDF over the same probabilities in index order (fp64) at the supplied uniforms [B]:
    token = first j with cumsum(p)[j] > u * sum(p).  Returns (tokens int64 [B], probs fp64 [B, V])."""
    z = logits.float() / temperature                                             # :230-231
    z = top_k_logits(z, top_k=top_k, top_p=top_p)                                # :232-233
    probs = F.softmax(z.double(), dim=-1)                                        # :234
    cdf = torch.cumsum(probs, dim=-1)
    target = uniforms.double().view(-1, 1) * cdf[:, -1:]
    tokens = (cdf <= target).sum(-1).clamp_max(logits.shape[-1] - 1)             # :235 (see above)
    return tokens, probs


# --------------------------------------------------------------------------- one position against a cache
# The generation loop feeds the whole token buffer through the model for every new token and keeps row
# context_length-1 of the output (Merak/inference/text_generation_inference.py:199-203,223).  The functions
# below compute that row for an HF Llama block (the model family the reference's examples wrap) from the new
# position alone plus the keys and values of the earlier ones; they are pinned against transformers' own
# LlamaDecoderLayer / LlamaModel run over the full sequence (tests/test_oracle_pins.py).
def rms_norm(x, weight, eps, residual=None):
    """HF LlamaRMSNorm.forward with the block's ``residual + hidden_states`` in front: returns (y, h)."""
    h = x if residual is None else residual + x
    hf = h.float()
    variance = hf.pow(2).mean(-1, keepdim=True)
    return weight * (hf * torch.rsqrt(variance + eps)).to(x.dtype), h


def rotate_half(x):
    """HF modeling_llama.rotate_half."""
    x1, x2 = x[..., : x.shape[-1] // 2], x[..., x.shape[-1] // 2:]
    return torch.cat((-x2, x1), dim=-1)


def rope_tables(head_dim, max_positions, theta=10000.0, dtype=torch.float32):
    """cos / sin [max_positions, head_dim] of HF LlamaRotaryEmbedding with the default rope type:
    inv_freq = theta^(-2i/d), angles = position x inv_freq, both halves of the last dim hold the same angles."""
    inv_freq = 1.0 / (theta ** (torch.arange(0, head_dim, 2, dtype=torch.int64).float() / head_dim))
    freqs = torch.outer(torch.arange(max_positions).float(), inv_freq)
    emb = torch.cat((freqs, freqs), dim=-1)
    return emb.cos().to(dtype), emb.sin().to(dtype)


def apply_rope(x, cos, sin):
    """HF apply_rotary_pos_emb for one position per row: x [B, heads, d], cos / sin [B, d]."""
    return x * cos[:, None, :] + rotate_half(x) * sin[:, None, :]


def attn_decode(q, k_cache, v_cache, lens, scale=None):
    """Grouped-query attention of one new position (HF eager_attention_forward with repeat_kv, no mask needed:
    every cached token is in the past): q [B, n_q, d], caches [B, n_kv, max_len, d], lens [B] -> [B, n_q, d]."""
    B, n_q, d = q.shape
    n_kv = k_cache.shape[1]
    g = n_q // n_kv
    scale = d ** -0.5 if scale is None else scale
    out = torch.zeros_like(q)
    for b in range(B):
        n = int(lens[b])
        if n == 0:
            continue
        k = k_cache[b, :, :n].repeat_interleave(g, dim=0)          # [n_q, n, d]
        v = v_cache[b, :, :n].repeat_interleave(g, dim=0)
        w = torch.einsum("hd,hnd->hn", q[b], k) * scale
        w = F.softmax(w, dim=-1, dtype=torch.float32).to(q.dtype)
        out[b] = torch.einsum("hn,hnd->hd", w, v)
    return out


def llama_block_step(x, residual, positions, lens, w, k_cache, v_cache, cos_table, sin_table, n_q_heads, eps):
    """One position per row through an HF LlamaDecoderLayer.  ``x`` is what the previous block's MLP returned
    (or the embedding), ``residual`` the stream it has to be added to (None for the first block); returns the
    same pair for the next block.  ``w``: input_norm, qkv [(n_q + 2 n_kv) d, H], o [H, n_q d],
    post_norm, gate_up [2 I, H] (gate rows first), down [H, I].  Writes the new key / value at ``positions``."""
    B = x.shape[0]
    n_kv, d = k_cache.shape[1], k_cache.shape[3]
    h, res = rms_norm(x, w["input_norm"], eps, residual)
    qkv = F.linear(h, w["qkv"]).view(B, n_q_heads + 2 * n_kv, d)
    cos, sin = cos_table[positions], sin_table[positions]
    q = apply_rope(qkv[:, :n_q_heads], cos, sin)
    k = apply_rope(qkv[:, n_q_heads:n_q_heads + n_kv], cos, sin)
    v = qkv[:, n_q_heads + n_kv:]
    for b in range(B):
        k_cache[b, :, positions[b]] = k[b]
        v_cache[b, :, positions[b]] = v[b]
    a = attn_decode(q, k_cache, v_cache, lens)
    o = F.linear(a.reshape(B, -1), w["o"])
    h2, res2 = rms_norm(o, w["post_norm"], eps, res)
    act = swiglu(F.linear(h2, w["gate_up"]))
    return F.linear(act, w["down"]), res2
