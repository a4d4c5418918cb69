"""CPU-only checks of the drop-in boundary: the C-ABI library loads, exports what the header declares,
validates arguments before any launch, and the Python front end keeps the reference's signature."""

import ctypes as C
import inspect
import os
import re

import pytest
import torch

from sample_efficient_gpt_amd import QKNormFlashAttnFunc, SelfDotProductAttnQKNorm, TritonFlashAttnQKNormFunc, _lib
from sample_efficient_gpt_amd import CONFIGS, make_inputs

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "segpt_attn.h")


@pytest.fixture(scope="module")
def lib():
    return _lib.load()


def _declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return re.findall(r"^\s*(?:const\s+)?[A-Za-z_][\w\s\*]*?\b(segpt_\w+)\s*\(", text, flags=re.M)


def test_library_exports_every_declared_symbol(lib):
    declared = _declared_functions()
    assert set(declared) == set(_lib.EXPORTED_SYMBOLS), declared
    for name in declared:
        assert getattr(lib, name) is not None
    assert lib.segpt_abi_version() == _lib.SEGPT_ABI_VERSION


def test_header_constants_match_binding():
    text = open(HEADER).read()
    consts = dict(re.findall(r"#define\s+(SEGPT_\w+)\s+(-?\d+)", text))
    assert int(consts["SEGPT_ABI_VERSION"]) == _lib.SEGPT_ABI_VERSION
    assert int(consts["SEGPT_DTYPE_BF16"]) == _lib.SEGPT_DTYPE_BF16
    assert int(consts["SEGPT_DTYPE_FP32"]) == _lib.SEGPT_DTYPE_FP32
    for name in ("SEGPT_FLAG_KV_PREPARED", "SEGPT_FLAG_RUNNING_MAX", "SEGPT_FLAG_DECODE", "SEGPT_FLAG_NO_NORM", "SEGPT_WS_KV", "SEGPT_WS_BWD"):
        assert int(consts[name]) == getattr(_lib, name), name
    stages = lambda prefix: [k for k, _ in sorted(((k, int(v)) for k, v in consts.items() if k.startswith(prefix)), key=lambda kv: kv[1])]
    assert [s.rsplit("_", 1)[1].lower() for s in stages("SEGPT_FWD_STAGE_")] == list(_lib.FWD_STAGES)
    assert [s.rsplit("_", 1)[1].lower() for s in stages("SEGPT_BWD_STAGE_")] == list(_lib.BWD_STAGES)
    # every error code has its own text
    texts = {_lib.strerror(int(v)) for k, v in consts.items() if k.startswith("SEGPT_E_")}
    assert len(texts) == len([k for k in consts if k.startswith("SEGPT_E_")])
    assert _lib.strerror(0) == "ok" and "HIP" in _lib.strerror(700)


def _valid_params(dtype=_lib.SEGPT_DTYPE_BF16, D=64):
    """Params with plausible (fake, never dereferenced) device addresses: validation happens on the host."""
    p = _lib.new_params()
    p.dtype = dtype
    p.B, p.H, p.Hkv, p.Sq, p.Sk, p.D = 2, 6, 2, 128, 128, D
    p.causal, p.q_start, p.gq_numel, p.gk_numel = 1, 0, D, 0
    p.eps, p.sm_scale, p.gate_scale = 1e-6, 0.125, 2.0
    fake = 0x10000
    for name in ("q", "o", "d_o", "dq"):
        setattr(p, name, _lib.Tensor4(fake, 6 * 128 * D, 128 * D, D))
    for name in ("k", "v", "dk", "dv"):
        setattr(p, name, _lib.Tensor4(fake, 2 * 128 * D, 128 * D, D))
    p.lse = p.g_q = p.dg_q = fake
    p.kv_workspace, p.kv_workspace_bytes = 0x40000, 1 << 30
    return p


def test_argument_errors_are_reported_before_any_launch(lib):
    # no GPU in this process: every call below must return from host-side validation
    assert lib.segpt_attn_fwd(None, None) == -1
    p = _valid_params()
    p.struct_bytes = 8
    assert lib.segpt_attn_fwd(p, None) == -2
    p = _valid_params(); p.dtype = 7
    assert lib.segpt_attn_fwd(p, None) == -3
    p = _valid_params(); p.Hkv = 4
    assert lib.segpt_attn_fwd(p, None) == -4
    p = _valid_params(); p.Sq = 0
    assert lib.segpt_attn_fwd(p, None) == -4
    p = _valid_params(); p.gq_numel = 3
    assert lib.segpt_attn_fwd(p, None) == -4
    p = _valid_params(D=48)
    assert lib.segpt_attn_fwd(p, None) == -5
    p = _valid_params(dtype=_lib.SEGPT_DTYPE_BF16, D=32)
    assert lib.segpt_attn_fwd(p, None) == -5
    p = _valid_params(); p.q.stride_s = 60
    assert lib.segpt_attn_fwd(p, None) == -6
    p = _valid_params(); p.k.stride_h = 7
    assert lib.segpt_attn_fwd(p, None) == -6
    # a bf16 row stride whose 256-row tile offsets would not fit 32 bits (the tile loads address rows that way)
    p = _valid_params(); p.q.stride_s = 1 << 23
    assert lib.segpt_attn_fwd(p, None) == -6
    # an OUTPUT view must not alias itself (a broadcast or overlapping view would make workgroups race)
    p = _valid_params(); p.o.stride_h = 0
    assert lib.segpt_attn_fwd(p, None) == -6
    p = _valid_params(); p.o.stride_b = 128 * 64  # batches overlap the heads
    assert lib.segpt_attn_fwd(p, None) == -6
    p = _valid_params(); p.workspace, p.workspace_bytes = 0x20000, 1 << 30
    p.dq.stride_b = 0
    assert lib.segpt_attn_bwd(p, None) == -6
    p = _valid_params(); p.workspace, p.workspace_bytes = 0x20000, 1 << 30
    p.dk = _lib.Tensor4(0x10000, 2 * 128 * 64, 64, 64)  # heads interleaved at the row pitch: rows collide
    assert lib.segpt_attn_bwd(p, None) == -6
    # the entry point with the library's own scratch validates the same way and needs no kv_workspace
    assert lib.segpt_attn_fwd_noalloc(None, None) == -1
    p = _valid_params(); p.kv_workspace, p.kv_workspace_bytes = None, 0; p.q.stride_s = 60
    assert lib.segpt_attn_fwd_noalloc(p, None) == -6
    p = _valid_params(); p.B, p.Sk = 4096, 4096  # 4096 * 2 * 4096 * 64 * 2 B of normalised keys
    assert lib.segpt_attn_fwd_noalloc(p, None) == _lib.SEGPT_E_SCRATCH_LIMIT
    p = _valid_params(); p.q_start = -1
    assert lib.segpt_attn_fwd(p, None) == -9
    p = _valid_params(); p.v.ptr = 0x10004
    assert lib.segpt_attn_fwd(p, None) == -10
    p = _valid_params(); p.q.ptr = None
    assert lib.segpt_attn_fwd(p, None) == -1
    p = _valid_params(); p.v_first = _lib.Tensor4(0x10000, 2 * 128 * 64, 128 * 64, 64)  # v_first without vr_coef
    assert lib.segpt_attn_fwd(p, None) == -8
    p = _valid_params(); p.kv_workspace = None
    assert lib.segpt_attn_fwd(p, None) == -7  # bf16 needs the key/value workspace
    p = _valid_params(); p.kv_workspace_bytes = lib.segpt_attn_workspace_bytes(p, _lib.SEGPT_WS_KV) - 1
    assert lib.segpt_attn_fwd(p, None) == -7
    p = _valid_params(); p.kv_workspace = 0x40010
    assert lib.segpt_attn_fwd(p, None) == -10
    assert lib.segpt_attn_fwd_stage(_valid_params(), 2, None) == -11
    assert lib.segpt_attn_bwd_stage(_valid_params(), 4, None) == -11
    # rotary tables: both or neither, aligned, long enough for the positions, bf16 only
    p = _valid_params(); p.rope_cos = 0x50000
    assert lib.segpt_attn_fwd(p, None) == -12
    p = _valid_params(); p.rope_cos, p.rope_sin, p.rope_len = 0x50000, 0x60000, 127  # Sq = Sk = 128 rows
    assert lib.segpt_attn_fwd(p, None) == -12
    p.rope_len, p.rope_q_pos0 = 128, 1
    assert lib.segpt_attn_fwd(p, None) == -12
    p.rope_q_pos0, p.rope_sin = 0, 0x60004
    assert lib.segpt_attn_fwd(p, None) == -12
    p = _valid_params(dtype=_lib.SEGPT_DTYPE_FP32); p.rope_cos, p.rope_sin, p.rope_len = 0x50000, 0x60000, p.Sk - 1
    assert lib.segpt_attn_fwd(p, None) == -12  # the fp32 path takes the tables too, under the same checks
    # backward-only checks
    p = _valid_params()
    assert lib.segpt_attn_bwd(p, None) == -7  # no workspace
    need = lib.segpt_attn_workspace_bytes(p, 1)
    p.workspace, p.workspace_bytes = 0x20000, need - 1
    assert lib.segpt_attn_bwd(p, None) == -7
    p = _valid_params(); p.dg_q = None
    assert lib.segpt_attn_bwd(p, None) == -1
    p = _valid_params(); p.gate = _lib.Tensor3(0x10000, 128 * 6, 6, 1)
    p.workspace, p.workspace_bytes = 0x20000, 1 << 30
    assert lib.segpt_attn_bwd(p, None) == -8  # gate without dgate slot


def test_workspace_bytes(lib):
    p = _valid_params()
    kv = lib.segpt_attn_workspace_bytes(p, _lib.SEGPT_WS_KV)
    assert kv >= 2 * 2 * 128 * 64 * 2 and kv % 256 == 0  # normalised keys [B,Hkv,Sk,D] bf16
    p.v_first = _lib.Tensor4(0x10000, 2 * 128 * 64, 128 * 64, 64)
    assert lib.segpt_attn_workspace_bytes(p, _lib.SEGPT_WS_KV) >= 2 * kv  # + mixed values
    assert lib.segpt_attn_workspace_bytes(_valid_params(dtype=_lib.SEGPT_DTYPE_FP32), _lib.SEGPT_WS_KV) == 0
    assert lib.segpt_attn_workspace_bytes(p, 2) == 0
    p = _valid_params()
    base = lib.segpt_attn_workspace_bytes(p, _lib.SEGPT_WS_BWD)
    rows = 2 * 6 * 128
    assert base >= rows * 4 and base % 256 == 0
    p.gate = _lib.Tensor3(0x10000, 128 * 6, 6, 1)
    assert lib.segpt_attn_workspace_bytes(p, 1) == base  # gate scale 2: the gate factor travels in the row statistics
    p.gate_scale = -1.0
    assert lib.segpt_attn_workspace_bytes(p, 1) == base + rows * 64 * 2  # a gate scale <= 0: + gated dO copy
    p32 = _valid_params(dtype=_lib.SEGPT_DTYPE_FP32)
    base32 = lib.segpt_attn_workspace_bytes(p32, 1)
    p32.gate = _lib.Tensor3(0x10000, 128 * 6, 6, 1)
    assert lib.segpt_attn_workspace_bytes(p32, 1) == base32 + rows * 64 * 4  # fp32 path: always
    bad = _valid_params(); bad.struct_bytes = 4
    assert lib.segpt_attn_workspace_bytes(bad, 1) == 0


def test_params_struct_matches_header_field_order():
    text = open(HEADER).read()
    body = text[text.index("typedef struct segpt_attn_params {"): text.index("} segpt_attn_params;")]
    body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
    names = []
    for decl in body.split(";"):
        decl = decl.strip()
        decl = decl.split("{")[-1].strip()
        if not decl:
            continue
        first, *rest = decl.split(",")
        names.append(re.findall(r"(\w+)\s*$", first.strip())[0])
        names += [r.strip().lstrip("*") for r in rest]
    assert names == [f[0] for f in _lib.AttnParams._fields_]


def test_function_signature_is_the_reference_one():
    # reference: forward(ctx, Q, K, V, gain, is_causal=True, q_start=0)  (triton_flash_attn_qknorm.py:264-272)
    sig = inspect.signature(QKNormFlashAttnFunc.forward)
    names = list(sig.parameters)
    assert names[:7] == ["ctx", "Q", "K", "V", "gain", "is_causal", "q_start"]
    assert sig.parameters["is_causal"].default is True and sig.parameters["q_start"].default == 0
    for extra in names[7:]:
        assert sig.parameters[extra].default is not inspect.Parameter.empty  # extras are optional
    assert issubclass(QKNormFlashAttnFunc, torch.autograd.Function)
    # the reference's own name: same positional signature, but its defaults are the reference KERNEL's formula
    # (eps = 1e-8 / d on the mean, logits gain * cos; triton_flash_attn_qknorm.py:67-91), resolved at call time
    assert issubclass(TritonFlashAttnQKNormFunc, QKNormFlashAttnFunc)
    ref_sig = inspect.signature(TritonFlashAttnQKNormFunc.forward)
    assert list(ref_sig.parameters) == names
    assert ref_sig.parameters["eps"].default is None and ref_sig.parameters["sm_scale"].default is None
    assert sig.parameters["eps"].default == 1e-6 and sig.parameters["sm_scale"].default is None


def test_function_asserts_like_the_reference_on_host_tensors():
    Q = torch.randn(2, 16, 64)
    with pytest.raises(AssertionError):  # `assert Q.is_cuda and Q.is_contiguous()`, :273
        QKNormFlashAttnFunc.apply(Q, Q, Q, torch.ones(1))


def test_module_interface():
    m = SelfDotProductAttnQKNorm(64)
    sd = m.state_dict()
    assert list(sd) == ["gain"] and sd["gain"].shape == (1,) and sd["gain"].dtype == torch.float32 and float(sd["gain"]) == 1.0
    sig = inspect.signature(m.forward)
    assert list(sig.parameters) == ["Q", "K", "V", "is_causal", "q_start"]


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "libsegpt_attn.so"))
    with pytest.raises(RuntimeError, match="no fallback"):
        _lib.load()


def test_input_generators_are_seeded_and_shaped():
    c = CONFIGS[1]
    a, b = make_inputs(c), make_inputs(c)
    assert all(torch.equal(a[k], b[k]) for k in a)
    assert a["q"].shape == (2, 4, 256, 64) and a["q"].dtype == torch.float32 and a["g_q"].shape == (64,)
    c4 = CONFIGS[4].scaled(S=64)
    x = make_inputs(c4)
    assert x["gate_logits"].shape == (2, 64, 18) and x["v_first"].shape == (2, 6, 64, 64)
    lam = float(x["vr_coef"][0])
    assert 0.3 <= lam <= 0.7 and abs(float(x["vr_coef"].sum()) - 1) < 1e-6
    assert CONFIGS[3].flops() == 7 * 8 * 18 * 2048 * 2048 * 64 and CONFIGS[2].flops() == 2 * 8 * 18 * 2048 * 2048 * 64


def test_library_op_is_registered_with_a_shape_only_implementation():
    """torch.ops.segpt.qknorm_attention: schema, fake (meta) forward and backward shapes, no kernel involved."""
    from sample_efficient_gpt_amd import qknorm_attention_op
    from torch._subclasses.fake_tensor import FakeTensorMode

    assert hasattr(torch.ops.segpt, "qknorm_attention") and hasattr(torch.ops.segpt, "qknorm_attention_backward")
    mk = lambda *s, dt=torch.bfloat16: torch.empty(*s, dtype=dt, device="meta", requires_grad=True)
    q, k, v, g = mk(2, 6, 96, 64), mk(2, 2, 96, 64), mk(2, 2, 96, 64), mk(64, dt=torch.float32)
    y, lse = qknorm_attention_op(q, k, v, g, None, return_lse=True)
    assert y.shape == q.shape and y.dtype == q.dtype and lse.shape == (2, 6, 96) and lse.dtype == torch.float32
    y.sum().backward()
    assert q.grad.shape == q.shape and k.grad.shape == k.shape and v.grad.shape == v.shape and g.grad.shape == g.shape
    with FakeTensorMode():  # what torch.compile sees: device tensors without storage
        dev = lambda *s, dt=torch.bfloat16: torch.empty(*s, dtype=dt, device="cuda")
        out = torch.ops.segpt.qknorm_attention(dev(1, 4, 50, 128), dev(1, 2, 70, 128), dev(1, 2, 70, 128), dev(1, dt=torch.float32),
                                               None, dev(1, 2, 70, 128), dev(2, dt=torch.float32), dev(1, 50, 4), 2.0, 1e-6, 0.1, True, 20, None, None, -1, 0, True, False, False)
        assert out[0].shape == (1, 4, 50, 128) and out[1].shape == (1, 4, 50)
        assert out[2].numel() == 2 * (2 * 70 * 128 * 2 + 255) // 256 * 256 or out[2].numel() >= 2 * 2 * 70 * 128 * 2


def test_plain_c_program_uses_the_library(tmp_path):
    """The boundary is a C ABI: a C99 program (gcc, no HIP or torch headers) includes the header, links the
    shared library and calls the entry points that need no GPU; its view of the struct matches the binding's."""
    import shutil
    import subprocess

    from sample_efficient_gpt_amd import _lib

    gcc = shutil.which("gcc")
    if gcc is None:
        pytest.skip("gcc not found")
    lib_path = _lib.LIB_PATH if hasattr(_lib, "LIB_PATH") else os.path.join(os.path.dirname(_lib.__file__), "libsegpt_attn.so")
    src = tmp_path / "t.c"
    src.write_text(r'''
#include <stdio.h>
#include <string.h>
#include "segpt_attn.h"
int main(void) {
  segpt_attn_params p;
  memset(&p, 0, sizeof p);
  p.struct_bytes = (int)sizeof p;
  p.dtype = SEGPT_DTYPE_BF16; p.B = 2; p.H = 6; p.Hkv = 2; p.Sq = 100; p.Sk = 100; p.D = 64;
  printf("%d %zu %zu %zu %d %s\n", segpt_abi_version(), sizeof p, segpt_attn_workspace_bytes(&p, SEGPT_WS_KV),
         segpt_attn_workspace_bytes(&p, SEGPT_WS_BWD), segpt_attn_fwd(&p, NULL), segpt_strerror(SEGPT_E_HEAD_DIM));
  return 0;
}
''')
    exe = tmp_path / "t"
    inc = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(_lib.__file__))), "include")
    subprocess.run([gcc, "-std=c99", "-Wall", "-Wextra", "-Werror", "-pedantic", f"-I{inc}", str(src), "-o", str(exe), lib_path,
                    f"-Wl,-rpath,{os.path.dirname(lib_path)}", "-Wl,-rpath,/opt/rocm/lib"], check=True)
    out = subprocess.run([str(exe)], check=True, stdout=subprocess.PIPE, text=True).stdout.split(maxsplit=5)
    lib = _lib.load()
    p = _lib.new_params()
    p.dtype, p.B, p.H, p.Hkv, p.Sq, p.Sk, p.D = _lib.SEGPT_DTYPE_BF16, 2, 6, 2, 100, 100, 64
    assert int(out[0]) == lib.segpt_abi_version()
    assert int(out[1]) == C.sizeof(p)
    assert int(out[2]) == lib.segpt_attn_workspace_bytes(p, _lib.SEGPT_WS_KV) == (2 * 2 * 100 * 64 * 2 + 255) // 256 * 256
    assert int(out[3]) == lib.segpt_attn_workspace_bytes(p, _lib.SEGPT_WS_BWD)
    assert int(out[4]) < 0  # argument error (no tensors bound), reported before any launch
    assert "head_dim" in out[5]
