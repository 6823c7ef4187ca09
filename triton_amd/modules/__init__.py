"""Generated-module counterparts: `get(variant, form, **consts)` or the per-variant files."""
from ._core import (FusedModule, RMSNorm, Attention, QKNormAttention, KeyFormerAttention, RoCoAttention,
                    PreNormBlock, DecodeVanilla, DecodeQKNorm, DecodeKeyFormer, DecodeRoCo, get)

__all__ = ["FusedModule", "RMSNorm", "Attention", "QKNormAttention", "KeyFormerAttention", "RoCoAttention",
           "PreNormBlock", "DecodeVanilla", "DecodeQKNorm", "DecodeKeyFormer", "DecodeRoCo", "get"]
