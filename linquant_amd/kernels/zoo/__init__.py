"""INT8 chunk forward kernels of the linear-recurrence zoo (HIP): linear attention with no / scalar decay,
GLA, DeltaNet / Gated DeltaNet, KDA.  Same call surface as linquant/kernels/zoo of the reference:
fp32 carry across chunks with an INT8 stored copy, round-half-away INT8 operands with per-role static scales,
fp32 C.B^T fed to an fp16 local product."""

from .gated_delta_rule import chunk_delta_int8
from .gla import chunk_gla_int8
from .kda import chunk_kda_int8
from .prologue import rotate_qkv, rotation_signs
from .simple_gla import chunk_simple_gla_int8

__all__ = ["chunk_simple_gla_int8", "chunk_gla_int8", "chunk_delta_int8", "chunk_kda_int8", "rotate_qkv", "rotation_signs"]
