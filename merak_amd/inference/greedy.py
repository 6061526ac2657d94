"""Greedy decode tail on the gfx950 kernels.

The reference's generation loop slices one position out of the logits and
takes ``torch.argmax(logits, dim=-1).view(-1)``
(Merak/inference/text_generation_inference.py:223,226-227).  Here the LM-head
product and the argmax are one kernel pass over the weight matrix: the [B, V]
logits are never written.  ``DecodeStep`` strings the single-token linears of
a Llama-shaped block in front of it (QKV, gate/up with SwiGLU, down), each a
GEMV that streams its weight once.
"""
from __future__ import annotations

from typing import Optional

import torch

from .. import ops


def greedy_from_logits(logits: torch.Tensor) -> torch.Tensor:
    """``torch.argmax(logits, dim=-1).view(-1)`` for materialised logits (first index on ties, NaN wins)."""
    return ops.argmax_rows(logits).view(-1)


def greedy_next_token(hidden: torch.Tensor, lm_head_weight: torch.Tensor,
                      workspace: Optional[torch.Tensor] = None) -> torch.Tensor:
    """argmax_n hidden[b] . lm_head_weight[n] for B <= 32 single-token rows, bf16."""
    idx, _ = ops.gemv_argmax(hidden, lm_head_weight, workspace)
    return idx


def top_k_logits(logits: torch.Tensor, top_k: int = 0, top_p: float = 0.0) -> torch.Tensor:
    """The reference's filter (text_generation_inference.py:35-69) on fp32 [B, V] logits: a new tensor with
    ``-inf`` where the reference writes its ``filter_value`` (the reference edits its argument in place)."""
    return ops.sample_top_k_top_p(logits, 1.0, top_k, top_p, None, want_filtered=True)[1]


def sample_next_token(logits: torch.Tensor, temperature: float = 1.0, top_k: int = 0, top_p: float = 0.0,
                      uniforms: Optional[torch.Tensor] = None, generator: Optional[torch.Generator] = None):
    """The live branch of the reference's loop (:229-235): ``logits.float() / temperature``, ``top_k_logits``,
    softmax, one multinomial draw per row.  The draw uses ``uniforms`` (fp32 [B] in [0, 1); drawn from
    ``generator`` or the default CUDA generator when omitted) instead of ``torch.multinomial``'s own stream."""
    if uniforms is None:
        uniforms = torch.rand((logits.shape[0],), device=logits.device, generator=generator)
    return ops.sample_top_k_top_p(logits, temperature, top_k, top_p, uniforms)[0]


class DecodeStep:
    """Single-token pass through QKV, gate/up (+SwiGLU), down and the LM head with fused argmax.

    Only the linears of the step live here (attention itself is outside the
    tensor-parallel layers); weights are the layers' own [out, in] bf16 tensors.
    """

    def __init__(self, w_qkv, w_gate_up, w_down, w_lm_head, max_batch: int = 32):
        self.w_qkv, self.w_gate_up, self.w_down, self.w_lm_head = w_qkv, w_gate_up, w_down, w_lm_head
        self.workspace = ops.argmax_workspace(max_batch, w_lm_head.shape[0], w_lm_head.shape[1], w_lm_head.device)
        # scratch of the linears that are cut along k at this batch size (the launches follow each other)
        self.max_batch = max_batch
        self._gemv_ws = {}

    def _ws(self, batch: int):
        if batch not in self._gemv_ws:
            need = [ops.gemv_workspace(batch, w.shape[0], w.shape[1], e, w.device)
                    for w, e in ((self.w_qkv, ops.EPI_NONE), (self.w_gate_up, ops.EPI_SWIGLU), (self.w_down, ops.EPI_NONE))]
            need = [t for t in need if t is not None]
            self._gemv_ws[batch] = max(need, key=lambda t: t.numel()) if need else None
        return self._gemv_ws[batch]

    def __call__(self, x: torch.Tensor):
        ws = self._ws(x.shape[0])
        # QKV and gate/up read the same rows: one call (one grid above 16 rows)
        qkv, h = ops.gemv_pair(x, self.w_qkv, self.w_gate_up, workspace=ws)
        out = ops.gemv(h, self.w_down, workspace=ws)
        token = greedy_next_token(out, self.w_lm_head, self.workspace)
        return qkv, out, token
