"""nn.Module with the interface and state-dict layout of the reference's QK-norm attention module."""

from __future__ import annotations

import torch
import torch.nn as nn

from .function import QKNormFlashAttnFunc


class SelfDotProductAttnQKNorm(nn.Module):
    """Same constructor, parameter (``gain`` of shape ``[1]``, fp32, init 1) and forward signature as
    sample_efficient_gpt/transformer/attention.py:30-80; the normalise + SDPA sequence of its forward
    is replaced by one fused kernel call.  Inputs are the flattened ``[(h b), S, d]`` tensors the
    reference's MultiHeadSelfAttention passes (attention.py:231-232); K/V may be left un-expanded when
    ``n_kv_heads`` is given.
    """

    def __init__(self, head_dim: int, n_kv_heads: int | None = None):
        super().__init__()
        self.head_dim = head_dim
        self.n_kv_heads = n_kv_heads
        self.gain = nn.Parameter(torch.tensor([1.0], dtype=torch.float32))

    def forward(self, Q, K, V, is_causal: bool = True, q_start: int = 0):
        lead = Q.shape[:-2]
        if Q.dim() > 3:  # "... seq_len d_k" inputs: fold the leading dims like the reference's kernels expect
            Q, K, V = (t.reshape(-1, *t.shape[-2:]) for t in (Q, K, V))
        n_kv = self.n_kv_heads if K.shape[0] != Q.shape[0] else None
        out = QKNormFlashAttnFunc.apply(Q.contiguous(), K.contiguous(), V.contiguous(), self.gain, is_causal, q_start,
                                        None, None, None, None, 2.0, n_kv)
        return out.reshape(*lead, *out.shape[-2:]) if len(lead) > 1 else out
