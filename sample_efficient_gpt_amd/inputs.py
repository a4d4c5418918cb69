"""Seeded synthetic inputs for the five benchmark / parity configurations.

Everything is drawn on the CPU in fp32 from ``torch.Generator().manual_seed(1000 + cfg)`` and then
cast, so that a CPU checker and the GPU kernels see identical bits.  Canonical layout:
q ``[B,H,S,D]``, k/v ``[B,Hkv,S,D]``.  The IMU-1 attention shape (18 query / 6 kv heads, head_dim 64)
is the reference model's, sample_efficient_gpt/configs/imu1_base.yaml:7-18.
"""

from __future__ import annotations

import dataclasses
import math

import torch


@dataclasses.dataclass(frozen=True)
class AttnConfig:
    cfg: int
    name: str
    B: int
    H: int
    Hkv: int
    S: int
    D: int
    dtype: torch.dtype
    backward: bool
    extras: bool = False       # per-head gate + value residual
    head_scales: bool = False  # per-(tensor, head) magnitude U(0.5, 2)
    eps: float = 1e-6
    gate_scale: float = 1.0

    @property
    def sm_scale(self) -> float:
        return 1.0 / math.sqrt(self.D)

    def flops(self, backward: bool | None = None) -> float:
        """Algorithmic FLOPs, causal FlashAttention convention: fwd 2*B*H*S^2*D, bwd 5*B*H*S^2*D."""
        backward = self.backward if backward is None else backward
        base = self.B * self.H * self.S * self.S * self.D
        return (7.0 if backward else 2.0) * base

    def scaled(self, **kw) -> "AttnConfig":
        return dataclasses.replace(self, **kw)


CONFIGS = {
    1: AttnConfig(1, "cpu_reference_fwd_fp32", 2, 4, 4, 256, 64, torch.float32, False),
    2: AttnConfig(2, "imu1_fwd", 8, 18, 6, 2048, 64, torch.bfloat16, False),
    3: AttnConfig(3, "imu1_fwd_bwd", 8, 18, 6, 2048, 64, torch.bfloat16, True),
    4: AttnConfig(4, "long_extras_fwd_bwd", 2, 18, 6, 8192, 64, torch.bfloat16, True, extras=True),
    5: AttnConfig(5, "wide_head_fwd_bwd", 4, 16, 4, 4096, 128, torch.bfloat16, True, head_scales=True),
}


def make_inputs(c: AttnConfig, device="cpu", seed: int | None = None) -> dict:
    """Returns a dict of tensors (cast to c.dtype where the op takes that dtype) on `device`.

    Keys: q, k, v, g_q, g_k, d_o and, with extras, gate_logits [B,S,H], v_first, vr_coef = (lam, 1-lam).
    """
    g = torch.Generator().manual_seed(1000 + c.cfg if seed is None else seed)

    def n(*shape):
        return torch.randn(*shape, generator=g, dtype=torch.float32)

    q, k, v = n(c.B, c.H, c.S, c.D), n(c.B, c.Hkv, c.S, c.D), n(c.B, c.Hkv, c.S, c.D)
    if c.head_scales:
        q = q * (0.5 + 1.5 * torch.rand(1, c.H, 1, 1, generator=g))
        k = k * (0.5 + 1.5 * torch.rand(1, c.Hkv, 1, 1, generator=g))
        v = v * (0.5 + 1.5 * torch.rand(1, c.Hkv, 1, 1, generator=g))
    out = {
        "q": q.to(c.dtype), "k": k.to(c.dtype), "v": v.to(c.dtype),
        "g_q": 1.0 + 0.02 * n(c.D), "g_k": 1.0 + 0.02 * n(c.D),
        "d_o": n(c.B, c.H, c.S, c.D).to(c.dtype),
    }
    if c.extras:
        lam = 0.3 + 0.4 * torch.rand(1, generator=g)
        out["gate_logits"] = n(c.B, c.S, c.H).to(c.dtype)
        out["v_first"] = n(c.B, c.Hkv, c.S, c.D).to(c.dtype)
        out["vr_coef"] = torch.cat([lam, 1.0 - lam]).to(torch.float32)
    return {k_: t.to(device) for k_, t in out.items()}
