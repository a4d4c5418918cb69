"""Shared helpers for the GPU parity tests: run the HIP op, run the CPU oracle, compare."""

from __future__ import annotations

import torch

from oracle import qknorm_attn_oracle as orc
from sample_efficient_gpt_amd import qknorm_attention

# north-star tolerances: bf16 kernels vs an fp32/fp64 reference: 2e-2 max-abs / 1e-2 relative; fp32 path: 1e-5
TOL = {torch.bfloat16: dict(atol=2e-2, rtol=1e-2), torch.float32: dict(atol=1e-5, rtol=1e-5)}


def gen(B, H, Hkv, Sq, Sk, D, dtype, *, extras=False, scalar_gain=False, no_gk=False, seed=0, head_scales=False):
    g = torch.Generator().manual_seed(seed)

    def n(*s):
        return torch.randn(*s, generator=g, dtype=torch.float32)

    x = {"q": n(B, H, Sq, D), "k": n(B, Hkv, Sk, D), "v": n(B, Hkv, Sk, D), "d_o": n(B, H, Sq, D)}
    if head_scales:
        x["q"] *= 0.5 + 1.5 * torch.rand(1, H, 1, 1, generator=g)
        x["k"] *= 0.5 + 1.5 * torch.rand(1, Hkv, 1, 1, generator=g)
        x["v"] *= 0.5 + 1.5 * torch.rand(1, Hkv, 1, 1, generator=g)
    x = {k: t.to(dtype) for k, t in x.items()}
    x["g_q"] = torch.tensor([1.3]) if scalar_gain else 1.0 + 0.02 * n(D)
    x["g_k"] = None if no_gk else 1.0 + 0.02 * n(D)
    if extras:
        x["gate_logits"] = n(B, Sq, H).to(dtype)
        x["v_first"] = n(B, Hkv, Sk, D).to(dtype)
        lam = 0.3 + 0.4 * torch.rand(1, generator=g)
        x["vr_coef"] = torch.cat([lam, 1 - lam])
    return x


def _split_rope(kw, device=None):
    """kw may carry rope=(cos, sin) (+ rope_q_pos0 / rope_k_pos0): returns the op's and the oracle's keyword sets."""
    kw = dict(kw)
    rope = kw.pop("rope", None)
    if rope is None:
        return kw, kw
    gpu_kw = dict(kw, rope_cos=rope[0].float().to(device) if device is not None else rope[0], rope_sin=rope[1].float().to(device) if device is not None else rope[1])
    return gpu_kw, dict(kw, rope=rope)


def run_gpu(x, device, *, backward=True, **kw):
    """Run the HIP op (and its backward) on `device`; returns CPU tensors."""
    kw, _ = _split_rope(kw, device)
    names = ["q", "k", "v", "g_q", "g_k", "v_first", "vr_coef", "gate_logits"]
    t = {n: (x[n].to(device).requires_grad_(backward) if x.get(n) is not None else None) for n in names}
    y, lse = qknorm_attention(t["q"], t["k"], t["v"], t["g_q"], t["g_k"], v_first=t["v_first"], vr_coef=t["vr_coef"],
                              gate_logits=t["gate_logits"], return_lse=True, **kw)
    out = {"y": y.detach().cpu(), "lse": lse.detach().cpu()}
    if backward:
        y.backward(x["d_o"].to(device))
        for n, gname in (("q", "dq"), ("k", "dk"), ("v", "dv"), ("g_q", "dg_q"), ("g_k", "dg_k"), ("v_first", "dv_first"),
                         ("vr_coef", "dvr_coef"), ("gate_logits", "dgate_logits")):
            if t[n] is not None:
                out[gname] = t[n].grad.detach().cpu()
    torch.cuda.synchronize()
    return out


def run_oracle(x, *, backward=True, odtype=torch.float64, **kw):
    """CPU oracle on the same bits, computed in `odtype`."""
    f = lambda n: None if x.get(n) is None else x[n].to(odtype)
    _, kw = _split_rope(kw)
    okw = dict(kw)
    if f("v_first") is not None:
        okw.update(v_first=f("v_first"), vr_coef=f("vr_coef"))
    if f("gate_logits") is not None:
        okw.update(gate_logits=f("gate_logits"))
    if not backward:
        y, lse, _, _ = orc.attention_forward(f("q"), f("k"), f("v"), f("g_q"), f("g_k"), **okw)
        return {"y": y, "lse": lse}
    return orc.attention_backward_autograd(f("q"), f("k"), f("v"), f("g_q"), f("g_k"), f("d_o"), **okw)


# Parameter gradients that are sums over every (batch, head, row): each summand carries its own bf16
# rounding noise, so the error of the sum scales with the norm of the summands, not with the (possibly
# cancelling) value of one entry.  For these the relative part of the tolerance is taken against the
# largest entry of the reference vector (norm-wise), everything else is compared element-wise.
REDUCED = ("dg_q", "dg_k", "dg", "dvr_coef")


def scalar_gain_scale(x, **kw):
    """Yardstick for the gradient of a SCALAR gain: it is the sum over d of the per-dimension scale
    gradients, whose rounding errors add up, so the relative tolerance is taken against
    sum_d |dg_d| of the oracle's vector-mode gradient rather than against the cancelled total."""
    D = x["q"].shape[-1]
    xv = dict(x)
    xv["g_q"] = x["g_q"].reshape(-1).expand(D).clone()
    ref = run_oracle(xv, **kw)
    return {"dg_q": float(ref["dg_q"].abs().sum())}


def value_residual_scale(x, ref):
    """Yardstick for the gradients of the two value-residual coefficients: dc1 = sum(dV' * v), dc2 = sum(dV' * v_first)
    over every key row and column; their bf16 rounding errors add up, so the relative tolerance refers to the
    sum of the magnitudes of the summands (dV' = dv / c1 from the oracle) instead of the cancelled total."""
    c1 = float(x["vr_coef"][0])
    dvm = ref["dv"].double() / c1
    return {"dvr_coef": float(max((dvm * x["v"].double()).abs().sum(), (dvm * x["v_first"].double()).abs().sum()))}


def compare(got, ref, dtype, names=None, label="", scales=None, outliers=None):
    """Asserts |got - ref| <= atol + rtol*|ref| for every output; returns {name: max_abs_err}.
    `scales` overrides the magnitude the relative part refers to for the named outputs.
    `outliers` = (fraction, factor): that fraction of a tensor's elements may exceed the bound, by at most
    `factor` (None: no element may)."""
    tol = TOL[dtype]
    errs = {}
    failures = []
    for n in (names or ref.keys()):
        r = ref[n].double()
        g = got[n].double().reshape(r.shape)
        if not torch.isfinite(g).all():
            failures.append(f"{label}{n}: non-finite values")
            continue
        err = (g - r).abs()
        scale = r.abs().max() if n in REDUCED else r.abs()
        if scales and n in scales:
            scale = max(float(r.abs().max()), scales[n])
        bound = tol["atol"] + tol["rtol"] * scale
        errs[n] = float(err.max())
        bad = err > bound
        if outliers is not None and bad.any() and int(bad.sum()) <= outliers[0] * bad.numel() and not (err > outliers[1] * bound).any():
            bad = bad & False
        if bad.any():
            failures.append(f"{label}{n}: {int(bad.sum())}/{bad.numel()} outside tolerance, max abs err {errs[n]:.3e} "
                            f"(ref max {float(r.abs().max()):.3e})")
    assert not failures, "; ".join(failures)
    return errs


def bf16_round(t):
    """Round-to-nearest-even to bf16, kept in the tensor's own (float64) dtype."""
    return t.to(torch.float32).to(torch.bfloat16).to(t.dtype)


def kernel_rounding_model(Q, K, V, g, dO, *, eps, sm_scale, causal, q_start):
    """The bf16 kernels' mathematics in float64 with a bf16 rounding at every point where the kernels hold a bf16
    value (csrc/fwd_mfma.hip, bwd_mfma.hip: the normalised operands Qhat and Khat, the probabilities and dS as MFMA
    operands, the saved output that delta is taken from) and exact arithmetic everywhere else.  Q [n,Sq,D], K, V
    [n,Sk,D], dO [n,Sq,D] hold bf16 values; g is the combined scale (1 or D elements).  Not a second oracle: it exists
    to say, per case, how far bf16 operand rounding moves the results away from the exact mathematics (the oracle), so
    that a test can demand the ordinary tolerance against THIS and report the distance to the oracle separately."""
    Q, K, V, dO, g = (t.double() for t in (Q, K, V, dO, g))
    n, Sq, D = Q.shape
    Sk = K.shape[1]
    log2e, ln2 = 1.4426950408889634, 0.6931471805599453
    a = torch.rsqrt((Q * Q).mean(-1, keepdim=True) + eps)
    b = torch.rsqrt((K * K).mean(-1, keepdim=True) + eps)
    qhat = bf16_round(sm_scale * log2e * a * Q * g)
    khat = bf16_round(b * K)
    s2 = qhat @ khat.transpose(1, 2)  # log2 units
    if causal:
        i = torch.arange(Sq).unsqueeze(1)
        j = torch.arange(Sk).unsqueeze(0)
        s2 = s2.masked_fill(j > i + q_start, float("-inf"))
    m = s2.max(-1, keepdim=True).values
    p = bf16_round(torch.exp2(s2 - m))
    l = p.sum(-1, keepdim=True)
    y = bf16_round((p @ V) / l)
    lse2 = m + torch.log2(l)
    # backward: P from the saved lse, delta from the saved (rounded) output
    P = torch.exp2(s2 - lse2)
    delta = (dO * y).sum(-1, keepdim=True)
    dP = dO @ V.transpose(1, 2)
    dS = P * (dP - delta)
    dv = bf16_round(P).transpose(1, 2) @ dO
    dSr = bf16_round(dS)
    T = dSr @ khat                      # dL/dQhat in units of the log2-scaled logits times ln2 ... see below
    dKhat = dSr.transpose(1, 2) @ qhat  # carries Qhat's sm_scale * log2e * g
    # dS is the gradient with respect to the NATURAL logit s = ln2 * s2, and s2 = qhat . khat, so
    # dL/dqhat = ln2 * dS khat and dL/dkhat = ln2 * dS^T qhat; qhat = f a q g with f = sm_scale * log2e
    u = (ln2 * sm_scale * log2e) * g * T                      # dL/d(a q)
    dq = a * (u - (a * a / D) * (u * Q).sum(-1, keepdim=True) * Q)
    dg = ((ln2 * sm_scale * log2e) * T * a * Q).sum((0, 1))  # per dimension; a scalar gain takes its sum
    W = ln2 * dKhat                                           # dL/dkhat
    dk = b * W - (b ** 3 / D) * (W * K).sum(-1, keepdim=True) * K
    return {"y": y, "dq": dq, "dk": dk, "dv": dv, "dg": dg}
