"""Drop-in module for the 'roco' variant in its prefill form with default constants: exposes the
reference's generated-module protocol (TritonGen.py:568-712) at module level, so a driver can
`importlib`-load this file where it would load a generated one."""
from ._core import get as _get

_module = _get("roco")
TENSOR_PARAMS = list(_module.TENSOR_PARAMS)
BLOCK_PARAMS = list(_module.BLOCK_PARAMS)
forward = _module.forward
