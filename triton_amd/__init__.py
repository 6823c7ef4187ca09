"""triton_amd: hand-written MI355X (gfx950) kernels for the fused operators that the
reference code generator emits -- RMSNorm, causal GQA/MQA flash attention, PreNorm,
QKNorm, KeyFormer and RoCo -- behind the reference's generated-module protocol
(`TENSOR_PARAMS`, `BLOCK_PARAMS`, in-place `forward`)."""
from . import _lib  # noqa: F401

__version__ = "0.1.0"
