"""segpt_attn_fwd_noalloc (the entry point that allocates nothing: its key/value scratch is a fixed array inside the
library's device image) against segpt_attn_fwd on the same operands, through the C ABI.  Same kernels, so the
results must be identical bit for bit; two calls in a row share the scratch, the second with a smaller input."""

import math

import pytest
import torch

from sample_efficient_gpt_amd import _lib
from sample_efficient_gpt_amd.function import _fill_common
from tests.parity_util import gen

pytestmark = pytest.mark.gpu


def _params(x, dev, y, lse, q_start=0, flags=0):
    t = {n: (None if x.get(n) is None else x[n].to(dev)) for n in ("q", "k", "v", "g_q", "g_k", "v_first", "vr_coef", "gate_logits")}
    f32 = lambda v: None if v is None else v.float().reshape(-1).contiguous()
    t["g_q"], t["g_k"], t["vr_coef"] = f32(t["g_q"]), f32(t["g_k"]), f32(t["vr_coef"])
    p = _lib.new_params()
    _fill_common(p, t["q"], t["k"], t["v"], y, lse, t["g_q"], t["g_k"], t["v_first"], t["vr_coef"], t["gate_logits"], 2.0,
                 1e-6, 1.0 / math.sqrt(t["q"].shape[-1]), True, q_start)
    p.flags = flags
    return p, t  # t keeps the device tensors alive


def _both(x, dev, q_start=0, flags=0):
    lib = _lib.load()
    B, H, Sq, D = x["q"].shape
    st = torch.cuda.current_stream(dev).cuda_stream
    outs = []
    for entry in ("segpt_attn_fwd", "segpt_attn_fwd_noalloc"):
        y = torch.full((B, H, Sq, D), float("nan"), dtype=torch.bfloat16, device=dev)
        lse = torch.full((B, H, Sq), float("nan"), dtype=torch.float32, device=dev)
        p, keep = _params(x, dev, y, lse, q_start, flags)
        if entry == "segpt_attn_fwd":
            ws = _lib.alloc_workspace(lib, p, _lib.SEGPT_WS_KV, dev)
            p.kv_workspace, p.kv_workspace_bytes = ws.data_ptr(), ws.numel()
        rc = getattr(lib, entry)(p, st)
        assert rc == 0, (entry, rc, _lib.strerror(rc))
        torch.cuda.synchronize()
        outs.append((y.cpu(), lse.cpu()))
        del keep
    (y0, l0), (y1, l1) = outs
    assert torch.isfinite(y1.float()).all() and torch.isfinite(l1).all()
    assert torch.equal(y0.view(torch.int16), y1.view(torch.int16)), "y differs between the two entry points"
    assert torch.equal(l0.view(torch.int32), l1.view(torch.int32)), "lse differs between the two entry points"


def test_noalloc_forward_matches_forward_twice_second_smaller(gpu_device):
    dev = gpu_device
    # first call: GQA 6:2 with gate + value residual (scratch holds normalised keys AND mixed values)
    _both(gen(2, 6, 2, 640, 640, 64, torch.bfloat16, extras=True, seed=11), dev)
    # second call, smaller, no extras: must not be affected by what the first left in the scratch
    _both(gen(1, 4, 2, 200, 200, 64, torch.bfloat16, seed=12), dev)
    # head_dim 128 and a decode-shaped call (scratch = split-key partial results)
    _both(gen(1, 4, 1, 130, 130, 128, torch.bfloat16, seed=13), dev)
    _both(gen(2, 6, 2, 1, 900, 64, torch.bfloat16, seed=14), dev, q_start=899, flags=_lib.SEGPT_FLAG_DECODE)


def test_noalloc_rejects_shapes_beyond_its_scratch(gpu_device):
    dev = gpu_device
    lib = _lib.load()
    x = gen(1, 1, 1, 64, 64, 64, torch.bfloat16, seed=1)
    y = torch.empty((1, 1, 64, 64), dtype=torch.bfloat16, device=dev)
    lse = torch.empty((1, 1, 64), dtype=torch.float32, device=dev)
    p, keep = _params(x, dev, y, lse)
    p.B, p.Hkv, p.H, p.Sk = 64, 8, 8, 4096  # 64*8*4096*64*2 B = 256 MiB of normalised keys: over the 16 MiB array
    need = lib.segpt_attn_workspace_bytes(p, _lib.SEGPT_WS_KV)
    assert need > _lib.SEGPT_NOALLOC_SCRATCH_BYTES
    rc = lib.segpt_attn_fwd_noalloc(p, torch.cuda.current_stream(dev).cuda_stream)  # rejected before any launch
    assert rc == _lib.SEGPT_E_SCRATCH_LIMIT
    assert "SEGPT_NOALLOC_SCRATCH_BYTES" in _lib.strerror(rc)


def test_noalloc_forward_in_a_captured_graph(gpu_device):
    """After one warm-up call outside capture (it looks the scratch address up), the entry point is plain kernel
    launches: captured into a HIP graph and replayed several times, with eager work on new inputs in between,
    every replay matches the eager result bit for bit."""
    dev = gpu_device
    lib = _lib.load()
    x = gen(2, 6, 2, 320, 320, 64, torch.bfloat16, extras=True, seed=21)
    B, H, Sq, D = x["q"].shape
    y = torch.zeros((B, H, Sq, D), dtype=torch.bfloat16, device=dev)
    lse = torch.zeros((B, H, Sq), dtype=torch.float32, device=dev)
    p, keep = _params(x, dev, y, lse)

    def call():
        rc = lib.segpt_attn_fwd_noalloc(p, torch.cuda.current_stream(dev).cuda_stream)
        assert rc == 0, (rc, _lib.strerror(rc))

    call()  # warm-up outside capture
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call()
    for seed in (31, 32, 33):
        new = gen(2, 6, 2, 320, 320, 64, torch.bfloat16, extras=True, seed=seed)
        for n in ("q", "k", "v", "v_first", "gate_logits"):
            keep[n].copy_(new[n].to(dev))  # same buffers, new contents
        call()  # eager, between the replays
        torch.cuda.synchronize()
        y_eager, lse_eager = y.clone(), lse.clone()
        y.zero_(); lse.zero_()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(y.view(torch.int16), y_eager.view(torch.int16)), seed
        assert torch.equal(lse.view(torch.int32), lse_eager.view(torch.int32)), seed
