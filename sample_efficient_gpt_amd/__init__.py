"""MI355X-native fused QK-norm causal GQA flash attention (forward + backward).

Drop-in for the attention hot path of thepowerfuldeez/sample_efficient_gpt:
``QKNormFlashAttnFunc`` mirrors the reference's ``TritonFlashAttnQKNormFunc`` call signature,
``SelfDotProductAttnQKNorm`` mirrors the live module, ``qknorm_attention`` is the same op on
canonical ``[B, H, S, D]`` views.  All compute runs in hand-written HIP kernels (gfx950) reached
through the C ABI of ``libsegpt_attn.so``; there is no fallback path.
"""

from .function import FlashAttnFunc, QKNormFlashAttnFunc, TritonFlashAttnQKNormFunc, qknorm_attention  # noqa: F401
from .module import KVCache, MultiHeadSelfAttention, SelfDotProductAttnQKNorm  # noqa: F401
from .library_op import qknorm_attention_op  # noqa: F401  (registers torch.ops.segpt.qknorm_attention)
from .inputs import CONFIGS, AttnConfig, make_inputs  # noqa: F401

# the reference's class names, so `from ... import TritonFlashAttnFunc` call sites keep working
# (TritonFlashAttnQKNormFunc is a subclass whose defaults are the reference kernel's own formula)
TritonFlashAttnFunc = FlashAttnFunc
