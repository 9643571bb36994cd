"""CPU oracle for the decode-step kernels between the int4 linears.  TEST INFRASTRUCTURE ONLY.

Nothing in the shipped package may import this module.

What it restates.  A decode step of the reference calls the Hugging Face ``LlamaModel`` on one
new token per row (``vrl/models/families/janus_pro/policy.py:673-678``).  The arithmetic between
the linears lives in that third-party model (``transformers`` 5.15 here; the reference pins no
version, ``pyproject.toml:28-33``), on bf16 tensors, every tensor op computing in fp32 and
rounding its result to bf16:

* ``LlamaDecoderLayer.forward``:  ``h = residual + sublayer_out``
* ``LlamaRMSNorm.forward``:       ``weight * (h.float() * rsqrt(mean(h.float()^2) + eps)).to(bf16)``
* ``apply_rotary_pos_emb``:       ``x * cos + rotate_half(x) * sin`` for q and k
* ``StaticLayer.update`` + ``sdpa_attention_forward``: write k, v at the new position, then
  ``softmax(q K^T * scaling + mask) V`` over the cache

Parity status.  The reference's tests replace the trunk by an identity stub
(``tests/models/test_janus_wrapper.py:30-57``) and hold no numeric vector for any of this:
PARITY UNPINNED against the reference.  Each function is pinned in ``tests/test_decode_oracle.py``
by running the library modules themselves on the CPU (``LlamaRMSNorm``, ``apply_rotary_pos_emb``,
``torch.nn.functional.scaled_dot_product_attention`` in float32 on the same bf16 values) and by
closed forms (a constant row normalises to the weight, rotation preserves the norm of each
(d, d + D/2) pair, one unmasked slot returns its value row, uniform scores average the values).

bf16 values travel as ``uint16`` bit patterns.
"""

from __future__ import annotations

import numpy as np

from .int4_oracle import bf16_bits_to_f32, f32_to_bf16_bits


def _rnd(v: np.ndarray) -> np.ndarray:
    """float32 -> nearest bf16 value, kept as float32."""
    return bf16_bits_to_f32(f32_to_bf16_bits(np.asarray(v, dtype=np.float32)))


def add_rmsnorm(x_bits, residual_bits, weight_bits, eps: float):
    """``(h_bits, y_bits)`` for rows ``x [M, K]``; ``residual_bits`` may be ``None`` (then h = x).

    The mean of squares is evaluated in float64 and rounded to float32 once (the squares of bf16
    values are exact in float32, so this is the correctly rounded mean any fp32 summation order
    approximates to a few units in the last place).
    """
    x = bf16_bits_to_f32(x_bits)
    h = x if residual_bits is None else _rnd(bf16_bits_to_f32(residual_bits) + x)
    K = h.shape[-1]
    var = (h.astype(np.float64) ** 2).sum(axis=-1, keepdims=True) * np.float64(np.float32(1.0) / np.float32(K))
    r = (np.float32(1.0) / np.sqrt((var.astype(np.float32) + np.float32(eps)).astype(np.float64))).astype(np.float32)
    xn = _rnd(h * r)
    y = _rnd(bf16_bits_to_f32(weight_bits)[None, :] * xn)
    return f32_to_bf16_bits(h), f32_to_bf16_bits(y)


def rotary(x_bits, cos_bits, sin_bits):
    """``apply_rotary_pos_emb`` for ``x [..., D]`` with table rows ``cos, sin [D]``: bf16 bits out."""
    x = bf16_bits_to_f32(x_bits)
    D = x.shape[-1]
    rot = np.concatenate([-x[..., D // 2:], x[..., :D // 2]], axis=-1)
    c, s = bf16_bits_to_f32(cos_bits), bf16_bits_to_f32(sin_bits)
    return f32_to_bf16_bits(_rnd(_rnd(x * c) + _rnd(rot * s)))


def rope_attn_decode(q_bits, k_bits, v_bits, k_cache_bits, v_cache_bits, cos_bits, sin_bits, mask,
                     position: int, n_heads: int, n_kv_heads: int, scaling: float):
    """One new token per row: returns ``(out float64 [M, H*D], k_cache_bits, v_cache_bits)``.

    ``q [M, H*D]``, ``k, v [M, Hkv*D]``, caches ``[M, Hkv, L, D]`` (copied, slot ``position``
    filled), tables ``[L, D]``, ``mask [M, L]`` (non-zero = attend).  Scores, softmax and the
    weighted sum are float64 over the bf16 values: the exact result any fp32 kernel approximates.
    """
    M = q_bits.shape[0]
    L, D = k_cache_bits.shape[2], k_cache_bits.shape[3]
    p = int(position)
    kc, vc = k_cache_bits.copy(), v_cache_bits.copy()
    q = rotary(q_bits.reshape(M, n_heads, D), cos_bits[p], sin_bits[p])
    kc[:, :, p, :] = rotary(k_bits.reshape(M, n_kv_heads, D), cos_bits[p], sin_bits[p])
    vc[:, :, p, :] = v_bits.reshape(M, n_kv_heads, D)
    group = n_heads // n_kv_heads
    qf = bf16_bits_to_f32(q).astype(np.float64)
    kf = bf16_bits_to_f32(kc[:, :, :p + 1, :]).astype(np.float64)
    vf = bf16_bits_to_f32(vc[:, :, :p + 1, :]).astype(np.float64)
    out = np.zeros((M, n_heads, D))
    for h in range(n_heads):
        hk = h // group
        s = np.einsum("md,mld->ml", qf[:, h], kf[:, hk]) * float(np.float32(scaling))
        s = np.where(np.asarray(mask)[:, :p + 1] != 0, s, -np.inf)
        s = s - s.max(axis=-1, keepdims=True)
        e = np.exp(s)
        out[:, h] = np.einsum("ml,mld->md", e / e.sum(axis=-1, keepdims=True), vf[:, hk])
    return out.reshape(M, n_heads * D), kc, vc


def lora_add(y_bits, x_bits, A, B, scaling: float, weights_fp32: bool):
    """``result = base + lora_B(lora_A(x)) * scaling`` of a PEFT LoRA wrapper, bf16 bits out.

    ``peft`` is not part of the reference tree (named only in an error message,
    ``vrl/models/families/janus_pro/policy.py:301-306``, ">=0.12"); this restates its published
    ``lora.Linear.forward``: with float32 adapter weights (its default, ``autocast_adapter_dtype``)
    the input is upcast, both products, the scaling and the sum with the bf16 base output are
    float32 and the result is rounded to bf16 once; with bf16 adapter weights every module output
    (``lora_A(x)``, ``lora_B(.)``, ``* scaling``, the sum) is rounded to bf16.  ``A [r, K]`` and
    ``B [N, r]`` are float arrays holding the weights' values.  Sums are float64 here.
    """
    x = bf16_bits_to_f32(x_bits).astype(np.float64)
    y = bf16_bits_to_f32(y_bits).astype(np.float64)
    t = x @ np.asarray(A, dtype=np.float64).T
    if not weights_fp32:
        t = _rnd(t).astype(np.float64)
    u = t @ np.asarray(B, dtype=np.float64).T
    if weights_fp32:
        delta = u * float(np.float32(scaling))
    else:
        delta = _rnd(_rnd(u).astype(np.float64) * float(np.float32(scaling))).astype(np.float64)
    return f32_to_bf16_bits((y + delta).astype(np.float32))
