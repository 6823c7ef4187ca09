"""Generated-module counterparts: `get(variant, form, **consts)` or the per-variant files."""
from ._core import (FusedModule, RMSNorm, Attention, QKNormAttention, KeyFormerAttention, RoCoAttention,
                    PreNormBlock, DecodeVanilla, DecodeQKNorm, DecodeKeyFormer, DecodeRoCo, get, roco_mean_std)

__all__ = ["FusedModule", "RMSNorm", "Attention", "QKNormAttention", "KeyFormerAttention", "RoCoAttention",
           "PreNormBlock", "DecodeVanilla", "DecodeQKNorm", "DecodeKeyFormer", "DecodeRoCo", "get", "roco_mean_std"]
