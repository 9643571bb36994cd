"""Host-side packed int4 format: packing, unpacking and the min/max quantiser.

Format (frozen here because the reference, guoriyue/VisionRL, ships no quantised
weights; its decode linears are bf16 ``nn.Linear`` modules reached from
``vrl/models/families/janus_pro/policy.py:673-678`` and ``:138-160``):

* ``qweight``  int32 ``[N, K/8]``: nibble ``i`` (bits ``4i..4i+3``) of word ``r`` is
  ``q[n, 8r+i]``, ``q`` in ``[0, 15]``.  ``q = 0..7`` packs to ``0x76543210``.
* ``scales``   bf16 ``[N, K/G]``: one scale per group of ``G`` consecutive ``k``.
* ``qzeros``   int32 ``[N, ceil(K/G/8)]``: zero-points in the same nibble order
  along the group axis; unused high nibbles of the last word are 0.
* ``w[n,k] = bf16((q[n,k] - z[n,k//G]) * s[n,k//G])``.

Everything here is loader glue that runs once per weight on whatever device
the tensors live on; the decode-time arithmetic is in the HIP library.
"""

from __future__ import annotations

import torch

NIBBLES_PER_WORD = 8


def _shifts(device) -> torch.Tensor:
    return torch.arange(0, 32, 4, dtype=torch.int32, device=device)


def pack_nibbles(q: torch.Tensor) -> torch.Tensor:
    """uint4 values ``[..., L]`` (any integer dtype) -> int32 ``[..., ceil(L/8)]``."""
    if q.dtype.is_floating_point:
        raise TypeError("pack_nibbles expects an integer tensor")
    if q.numel() and (int(q.min()) < 0 or int(q.max()) > 15):
        raise ValueError("nibble values must lie in [0, 15]")
    L = q.shape[-1]
    words = (L + NIBBLES_PER_WORD - 1) // NIBBLES_PER_WORD
    padded = torch.zeros(*q.shape[:-1], words * NIBBLES_PER_WORD, dtype=torch.int64, device=q.device)
    padded[..., :L] = q.to(torch.int64)
    padded = padded.reshape(*q.shape[:-1], words, NIBBLES_PER_WORD)
    word = (padded << _shifts(q.device).to(torch.int64)).sum(dim=-1)
    # two's-complement wrap of the top nibble into int32
    word = torch.where(word >= 2 ** 31, word - 2 ** 32, word)
    return word.to(torch.int32).contiguous()


def unpack_nibbles(packed: torch.Tensor, length: int) -> torch.Tensor:
    """int32 ``[..., W]`` -> uint8 ``[..., length]``; inverse of :func:`pack_nibbles`."""
    if packed.dtype != torch.int32:
        raise TypeError("packed nibbles must be int32")
    if length > packed.shape[-1] * NIBBLES_PER_WORD:
        raise ValueError("length exceeds packed capacity")
    nib = (packed.unsqueeze(-1) >> _shifts(packed.device)) & 0xF
    nib = nib.reshape(*packed.shape[:-1], packed.shape[-1] * NIBBLES_PER_WORD)
    return nib[..., :length].to(torch.uint8)


def check_packed(qweight: torch.Tensor, scales: torch.Tensor, qzeros: torch.Tensor,
                 group_size: int) -> tuple[int, int, int]:
    """Validate a packed operand triple; returns ``(N, K, groups)``."""
    if qweight.dtype != torch.int32 or qzeros.dtype != torch.int32:
        raise TypeError("qweight and qzeros must be int32")
    if scales.dtype != torch.bfloat16:
        raise TypeError("scales must be bfloat16")
    if qweight.dim() != 2 or scales.dim() != 2 or qzeros.dim() != 2:
        raise ValueError("qweight, scales and qzeros must be 2-D")
    G = int(group_size)
    if G <= 0 or G % NIBBLES_PER_WORD != 0:
        raise ValueError("group_size must be a positive multiple of 8")
    N, kw = qweight.shape
    K = kw * NIBBLES_PER_WORD
    if K == 0 or K % G != 0:
        raise ValueError(f"K={K} must be a positive multiple of group_size={G}")
    groups = K // G
    if tuple(scales.shape) != (N, groups):
        raise ValueError(f"scales must be [{N}, {groups}], got {tuple(scales.shape)}")
    zw = (groups + NIBBLES_PER_WORD - 1) // NIBBLES_PER_WORD
    if tuple(qzeros.shape) != (N, zw):
        raise ValueError(f"qzeros must be [{N}, {zw}], got {tuple(qzeros.shape)}")
    return N, K, groups


def quantize_minmax(weight: torch.Tensor, group_size: int):
    """Asymmetric min/max uint4 quantiser, one (scale, zero) per K-group.

    The range of each group is widened to contain 0 so that a zero weight stays
    exactly zero.  ``s = bf16((max - min) / 15)`` (1 for an all-zero group),
    ``z = clamp(round(-min / s), 0, 15)``, ``q = clamp(round(w / s) + z, 0, 15)``,
    computed in fp32 with the bf16-rounded scale (the one the kernel will use).

    Returns ``(qweight int32 [N,K/8], scales bf16 [N,K/G], qzeros int32 [N,ceil(K/G/8)])``.
    """
    if weight.dim() != 2:
        raise ValueError("weight must be [N, K]")
    N, K = weight.shape
    G = int(group_size)
    if G <= 0 or G % NIBBLES_PER_WORD != 0 or K % G != 0:
        raise ValueError("group_size must be a multiple of 8 that divides K")
    g = weight.detach().to(torch.float32).reshape(N, K // G, G)
    lo = g.amin(dim=-1).clamp(max=0.0)
    hi = g.amax(dim=-1).clamp(min=0.0)
    span = hi - lo
    raw = torch.where(span > 0, span / 15.0, torch.ones_like(span))
    scales = raw.to(torch.bfloat16)
    s = scales.to(torch.float32)
    z = torch.clamp(torch.round(-lo / s), 0, 15)
    q = torch.clamp(torch.round(g / s.unsqueeze(-1)) + z.unsqueeze(-1), 0, 15)
    qweight = pack_nibbles(q.reshape(N, K).to(torch.int32))
    qzeros = pack_nibbles(z.to(torch.int32))
    return qweight, scales.contiguous(), qzeros


def algorithmic_bytes(M: int, K: int, N: int, G: int, fused_gate_up: bool = False) -> int:
    """Bytes one call must move: 4-bit weights, bf16 scales, 4-bit zeros, bf16 x and y."""
    groups = K // G
    out_cols = N // 2 if fused_gate_up else N
    return K * N // 2 + groups * N * 2 + groups * N // 2 + M * K * 2 + M * out_cols * 2
