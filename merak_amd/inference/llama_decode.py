"""One new position per sequence through a Llama-shaped model with a key/value cache.

The reference's generation loop pushes the whole token buffer through the
model for every new token and keeps row ``context_length - 1`` of the output
(Merak/inference/text_generation_inference.py:199-203,223).  A causal model
gives the same row from the new position alone once the keys and values of
the earlier positions are kept, which turns every linear of the block into a
GEMV that streams its weight once and the attention into one pass over the
cache.  ``LlamaDecoder.step`` is that row; the greedy pick (:226-227) or the
sampling tail (:229-235) follows it.

Weights are the tensor-parallel layers' own tensors: the fused QKV and
gate/up column-parallel weights ([out, in], q heads / k heads / v heads and
gate rows / up rows stacked along ``out``) and the row-parallel ``o`` and
``down`` weights.
"""
from __future__ import annotations

import math
from dataclasses import dataclass
from typing import List, Optional

import torch

from .. import ops
from .greedy import greedy_next_token


def rope_tables(head_dim: int, max_positions: int, theta: float = 10000.0, scaling: Optional[dict] = None,
                dtype: torch.dtype = torch.float32, device=None):
    """cos / sin tables [max_positions, head_dim] of HF ``LlamaRotaryEmbedding``: default rope type, or
    ``scaling = {"rope_type": "llama3", "factor", "low_freq_factor", "high_freq_factor",
    "original_max_position_embeddings"}`` (the Llama-3.1 frequency rescale).  Computed in fp32, then cast."""
    inv_freq = 1.0 / (theta ** (torch.arange(0, head_dim, 2, dtype=torch.int64).float() / head_dim))
    if scaling is not None and scaling.get("rope_type", "default") != "default":
        if scaling["rope_type"] != "llama3":
            raise NotImplementedError(f"rope_type {scaling['rope_type']!r}")
        factor, low, high = scaling["factor"], scaling["low_freq_factor"], scaling["high_freq_factor"]
        old_len = scaling["original_max_position_embeddings"]
        wavelen = 2 * math.pi / inv_freq
        scaled = torch.where(wavelen > old_len / low, inv_freq / factor, inv_freq)
        smooth = (old_len / wavelen - low) / (high - low)
        mid = (1 - smooth) * scaled / factor + smooth * scaled
        is_mid = ~(wavelen < old_len / high) & ~(wavelen > old_len / low)
        inv_freq = torch.where(is_mid, mid, scaled)
    freqs = torch.outer(torch.arange(max_positions).float(), inv_freq)
    emb = torch.cat((freqs, freqs), dim=-1)
    return emb.cos().to(dtype=dtype, device=device), emb.sin().to(dtype=dtype, device=device)


@dataclass
class LlamaBlockWeights:
    input_norm: torch.Tensor   # [H]
    qkv: torch.Tensor          # [(n_q + 2 n_kv) * head_dim, H]
    o: torch.Tensor            # [H, n_q * head_dim]
    post_norm: torch.Tensor    # [H]
    gate_up: torch.Tensor      # [2 I, H]: gate rows, then up rows
    down: torch.Tensor         # [H, I]


class LlamaDecoder:
    """Decode-only runner: ``step(tokens)`` appends one token per sequence and returns the next one.

    ``batch`` sequences share one cache allocation [batch, n_kv_heads, max_len, head_dim] per layer; every
    sequence has its own length (``self.lens``, on the device, so a step never synchronises with the host)."""

    def __init__(self, embed: torch.Tensor, blocks: List[LlamaBlockWeights], final_norm: torch.Tensor,
                 lm_head: torch.Tensor, n_q_heads: int, n_kv_heads: int, head_dim: int = 128, eps: float = 1e-5,
                 rope_theta: float = 10000.0, rope_scaling: Optional[dict] = None, max_len: int = 4096,
                 batch: int = 1, fused: Optional[bool] = None):
        dev, dt = lm_head.device, lm_head.dtype
        self.embed, self.blocks, self.final_norm, self.lm_head = embed, blocks, final_norm, lm_head
        self.n_q, self.n_kv, self.head_dim, self.eps = n_q_heads, n_kv_heads, head_dim, eps
        self.max_len, self.batch = max_len, batch
        # norms and residual adds inside the linears: the norm prologue keeps the batch's normalised rows in LDS
        can_fuse = ops.gemv_norm_fits(batch, embed.shape[1])
        if fused and not can_fuse:
            raise ValueError(f"fused=True needs batch x hidden <= 8 x 4096 and hidden % 512 == 0, got {batch} x {embed.shape[1]}")
        self.fused = can_fuse if fused is None else bool(fused)
        self.cos, self.sin = rope_tables(head_dim, max_len, rope_theta, rope_scaling, dtype=dt, device=dev)
        self.k_cache = [torch.zeros((batch, n_kv_heads, max_len, head_dim), dtype=dt, device=dev) for _ in blocks]
        self.v_cache = [torch.zeros((batch, n_kv_heads, max_len, head_dim), dtype=dt, device=dev) for _ in blocks]
        self.lens = torch.zeros((batch,), dtype=torch.int64, device=dev)
        self.host_len_bound = 0           # upper bound of self.lens kept on the host
        self.argmax_ws = ops.argmax_workspace(batch, lm_head.shape[0], lm_head.shape[1], dev)
        # the number of splits, and with it the need, does not shrink when the length bound grows
        self.attn_ws = ops.attn_workspace(batch, n_q_heads, n_kv_heads, max_len, dev)
        w0 = blocks[0]
        need = [ops.gemv_workspace(batch, w.shape[0], w.shape[1], e, dev)
                for w, e in ((w0.qkv, ops.EPI_NONE), (w0.o, ops.EPI_NONE), (w0.gate_up, ops.EPI_SWIGLU),
                             (w0.down, ops.EPI_NONE), (lm_head, ops.EPI_NONE))]
        need = [t for t in need if t is not None]
        self.gemv_ws = max(need, key=lambda t: t.numel()) if need else None

    @classmethod
    def from_hf(cls, model, max_len: int = 4096, batch: int = 1, fused: Optional[bool] = None):
        """From a ``transformers`` ``LlamaForCausalLM`` (weights are concatenated once, not shared)."""
        cfg = model.config
        blocks = []
        for layer in model.model.layers:
            a, m = layer.self_attn, layer.mlp
            blocks.append(LlamaBlockWeights(
                layer.input_layernorm.weight.data,
                torch.cat([a.q_proj.weight.data, a.k_proj.weight.data, a.v_proj.weight.data]).contiguous(),
                a.o_proj.weight.data.contiguous(), layer.post_attention_layernorm.weight.data,
                torch.cat([m.gate_proj.weight.data, m.up_proj.weight.data]).contiguous(),
                m.down_proj.weight.data.contiguous()))
        rp = getattr(cfg, "rope_parameters", None) or getattr(cfg, "rope_scaling", None) or {}
        theta = rp.get("rope_theta", getattr(cfg, "rope_theta", 10000.0))
        scaling = rp if rp.get("rope_type", "default") != "default" else None
        head_dim = getattr(cfg, "head_dim", None) or cfg.hidden_size // cfg.num_attention_heads
        return cls(model.model.embed_tokens.weight.data, blocks, model.model.norm.weight.data,
                   model.lm_head.weight.data, cfg.num_attention_heads, cfg.num_key_value_heads, head_dim,
                   cfg.rms_norm_eps, theta, scaling, max_len, batch, fused)

    def reset(self):
        self.lens.zero_()
        self.host_len_bound = 0

    def _hidden(self, tokens: torch.Tensor, len_bound: int) -> torch.Tensor:
        if self.fused:
            return self._hidden_fused(tokens, len_bound)
        positions = self.lens             # tokens cached so far = position of the new one
        x = ops.embedding_gather(tokens, self.embed, 0, self.embed.shape[0])
        residual = None
        B = x.shape[0]
        for w, kc, vc in zip(self.blocks, self.k_cache, self.v_cache):
            h, residual = ops.rmsnorm(x, w.input_norm, self.eps, residual, want_residual=True)
            qkv = ops.gemv(h, w.qkv, workspace=self.gemv_ws)
            a = ops.attn_decode_append(qkv, self.cos, self.sin, positions, kc, vc, self.n_q, len_bound=len_bound,
                                       workspace=self.attn_ws)
            o = ops.gemv(a.view(B, -1), w.o, workspace=self.gemv_ws)
            h, residual = ops.rmsnorm(o, w.post_norm, self.eps, residual, want_residual=True)
            act = ops.gemv(h, w.gate_up, None, ops.EPI_SWIGLU, workspace=self.gemv_ws)
            x = ops.gemv(act, w.down, workspace=self.gemv_ws)
        self.lens += 1
        return ops.rmsnorm(x, self.final_norm, self.eps, residual)

    def _hidden_fused(self, tokens: torch.Tensor, len_bound: int) -> torch.Tensor:
        """Five launches per block: the two RMSNorms ride in the QKV and gate/up products (the o and down products
        hand them the sums of squares of the residual stream they write), the residual adds in the o and down
        products.  The rounding steps are those of the seven-launch form."""
        positions = self.lens
        x = ops.embedding_gather(tokens, self.embed, 0, self.embed.shape[0])      # the residual stream
        B = x.shape[0]
        ss = None
        for w, kc, vc in zip(self.blocks, self.k_cache, self.v_cache):
            if ss is None:      # first block: the stream comes from the embedding, nobody has summed its squares
                qkv = ops.gemv(ops.rmsnorm(x, w.input_norm, self.eps), w.qkv, workspace=self.gemv_ws)
            else:
                qkv = ops.gemv_fused(x, w.qkv, norm_weight=w.input_norm, sumsq_in=ss, eps=self.eps)
            a = ops.attn_decode_append(qkv, self.cos, self.sin, positions, kc, vc, self.n_q, len_bound=len_bound,
                                       workspace=self.attn_ws)
            x, ss = ops.gemv_fused(a.view(B, -1), w.o, residual=x, want_sumsq=True, workspace=self.gemv_ws)
            act = ops.gemv_fused(x, w.gate_up, None, ops.EPI_SWIGLU, norm_weight=w.post_norm, sumsq_in=ss, eps=self.eps)
            x, ss = ops.gemv_fused(act, w.down, residual=x, want_sumsq=True, workspace=self.gemv_ws)
        self.lens += 1
        return ops.rmsnorm(x, self.final_norm, self.eps)

    def capture(self):
        """Records one step (all blocks, final norm, LM head with argmax) into a HIP graph; ``hidden`` / ``logits``
        / ``step`` replay it from then on, which takes the ~230 launches of a step off the Python path.
        Sequence lengths live on the device, so the same graph serves every later position; the attention is
        recorded with the split count of a full cache."""
        dev = self.lm_head.device
        self._tokens_in = torch.zeros((self.batch,), dtype=torch.int64, device=dev)
        saved = self.lens.clone()
        cur = torch.cuda.current_stream(dev)
        side = torch.cuda.Stream(dev)
        side.wait_stream(cur)
        with torch.cuda.stream(side):       # two real steps first (they write cache rows that later tokens overwrite)
            for _ in range(2):
                greedy_next_token(self._hidden(self._tokens_in, self.max_len), self.lm_head, self.argmax_ws)
            self.lens.copy_(saved)
        cur.wait_stream(side)
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            self._hidden_out = self._hidden(self._tokens_in, self.max_len)
            self._token_out = greedy_next_token(self._hidden_out, self.lm_head, self.argmax_ws)
        self._graph = graph

    def hidden(self, tokens: torch.Tensor) -> torch.Tensor:
        """Appends ``tokens`` (int64 [batch]) and returns the final-norm output [batch, H] of their position."""
        if self.host_len_bound >= self.max_len:
            raise RuntimeError(f"key/value cache full ({self.max_len} positions)")
        self.host_len_bound += 1
        if getattr(self, "_graph", None) is not None:
            self._tokens_in.copy_(tokens)
            self._graph.replay()
            return self._hidden_out
        return self._hidden(tokens, self.host_len_bound)

    def logits(self, tokens: torch.Tensor) -> torch.Tensor:
        """The row the reference slices out at :223 (fp32 accumulation, model dtype)."""
        return ops.gemv(self.hidden(tokens), self.lm_head, workspace=self.gemv_ws)

    def step(self, tokens: torch.Tensor) -> torch.Tensor:
        """Greedy next token per sequence (:226-227); the [batch, vocab] logits are never written."""
        h = self.hidden(tokens)
        if getattr(self, "_graph", None) is not None:
            return self._token_out.clone()
        return greedy_next_token(h, self.lm_head, self.argmax_ws)
