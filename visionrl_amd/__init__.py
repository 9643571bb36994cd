"""MI355X-native int4 weight-only decode linears for autoregressive rollout.

``ops``          torch operators over the HIP library (``vrl_hip::int4_gemv`` ...)
``int4_format``  packed-nibble format, packer and min/max quantiser (loader glue)
``linear``       ``Int4Linear`` drop-in for the policy's ``nn.Linear`` layers
``policy_glue``  swaps the decode linears of a Janus-Pro style policy
``ar_decode``    ``sample_image_tokens`` / step API over a static KV cache, one recorded step per token
``decode_step``  one decode step of the int4 trunk as a fixed list of native launches
"""

from .int4_format import (algorithmic_bytes, check_packed, pack_nibbles, quantize_minmax,
                          unpack_nibbles)
from ._lib import Int4LibraryError

__all__ = [
    "Int4LibraryError",
    "algorithmic_bytes",
    "check_packed",
    "pack_nibbles",
    "quantize_minmax",
    "unpack_nibbles",
]
