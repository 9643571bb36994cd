"""Pins ``oracle/decode_oracle.py`` against the library modules it restates (run on the CPU) and
against closed forms; the reference holds no numeric vector for these ops."""

import numpy as np
import pytest
import torch

from oracle import decode_oracle as d
from oracle import int4_oracle as o
from tests._util import bf16_to_bits, bits_to_bf16


def rand_bits(rng, shape, scale=1.0):
    return o.f32_to_bf16_bits((rng.standard_normal(shape) * scale).astype(np.float32))


def ulp_distance(a_bits, b_bits):
    """Distance in bf16 steps between two arrays of finite bf16 patterns."""
    def key(b):
        b = b.astype(np.int32)
        return np.where(b & 0x8000, -(b & 0x7FFF), b & 0x7FFF)
    return np.abs(key(a_bits) - key(b_bits))


def within_one_step_of(got_bits, want_bits, operand_bits):
    """|got - want| <= one bf16 step at the magnitude of the larger of result and operand (a sum that
    cancels is only as exact as its operands' steps); returns the fraction of differing elements."""
    got, want = o.bf16_bits_to_f32(got_bits).astype(np.float64), o.bf16_bits_to_f32(want_bits).astype(np.float64)
    ref = np.maximum(np.abs(want), np.abs(o.bf16_bits_to_f32(operand_bits).astype(np.float64)))
    assert (np.abs(got - want) <= o.bf16_ulp(ref.astype(np.float32))).all(), np.abs(got - want).max()
    return float((got_bits != want_bits).mean())


@pytest.mark.parametrize("M,K,with_residual", [(2, 2048, True), (3, 256, False), (5, 4096, True), (1, 3072, True)])
def test_add_rmsnorm_matches_llama_rmsnorm(M, K, with_residual):
    from transformers.models.llama.modeling_llama import LlamaRMSNorm

    rng = np.random.default_rng(K + M)
    x, res, w = rand_bits(rng, (M, K)), rand_bits(rng, (M, K), 3.0), rand_bits(rng, (K,), 0.5)
    norm = LlamaRMSNorm(K, eps=1e-6).to(torch.bfloat16)
    with torch.no_grad():
        norm.weight.copy_(bits_to_bf16(w))
        h = bits_to_bf16(res) + bits_to_bf16(x) if with_residual else bits_to_bf16(x)
        want = norm(h)
    h_bits, y_bits = d.add_rmsnorm(x, res if with_residual else None, w, 1e-6)
    assert (h_bits == bf16_to_bits(h)).all()
    dist = ulp_distance(y_bits, bf16_to_bits(want))
    # the library sums the squares in float32 in its own order: a rounding of the normalised value
    # may flip for a handful of elements, never by more than one step
    assert dist.max() <= 1 and (dist > 0).mean() < 2e-3


def test_add_rmsnorm_closed_forms():
    K = 512
    w = rand_bits(np.random.default_rng(0), (K,))
    x = o.f32_to_bf16_bits(np.full((1, K), -3.0, dtype=np.float32))
    _, y = d.add_rmsnorm(x, None, w, 0.0)   # a constant row normalises to -1: y = -weight
    assert (y[0] == (w ^ 0x8000)).all()
    big = o.f32_to_bf16_bits(np.full((1, K), 2.0 ** 60, dtype=np.float32))   # squares overflow nothing in fp32
    _, y = d.add_rmsnorm(big, None, w, 1e-6)
    assert (y[0] == w).all()
    # the add is rounded to bf16 before the norm sees it
    a = o.f32_to_bf16_bits(np.full((1, K), 1.0, dtype=np.float32))
    b = o.f32_to_bf16_bits(np.full((1, K), 2.0 ** -9, dtype=np.float32))   # 1 + 2^-9 rounds back to 1
    h, _ = d.add_rmsnorm(a, b, w, 1e-6)
    assert (h == a).all()


@pytest.mark.parametrize("D", [64, 128])
def test_rotary_matches_apply_rotary_pos_emb(D):
    from transformers.models.llama.modeling_llama import apply_rotary_pos_emb

    rng = np.random.default_rng(D)
    q, k = rand_bits(rng, (3, 4, 1, D)), rand_bits(rng, (3, 4, 1, D))
    ang = rng.uniform(0, 600, size=(1, D // 2)).astype(np.float32)
    emb = np.concatenate([ang, ang], axis=-1)
    cos, sin = o.f32_to_bf16_bits(np.cos(emb)), o.f32_to_bf16_bits(np.sin(emb))
    qe, ke = apply_rotary_pos_emb(bits_to_bf16(q), bits_to_bf16(k), bits_to_bf16(cos)[None], bits_to_bf16(sin)[None])
    assert (d.rotary(q, cos[0], sin[0]) == bf16_to_bits(qe)).all()
    assert (d.rotary(k, cos[0], sin[0]) == bf16_to_bits(ke)).all()
    # a rotation: each (d, d + D/2) pair keeps its length up to the bf16 roundings
    x = o.bf16_bits_to_f32(q).astype(np.float64)
    y = o.bf16_bits_to_f32(d.rotary(q, cos[0], sin[0])).astype(np.float64)
    n0 = np.hypot(x[..., :D // 2], x[..., D // 2:])
    n1 = np.hypot(y[..., :D // 2], y[..., D // 2:])
    assert np.abs(n1 - n0).max() <= 2 ** -6 * n0.max()


def attn_case(seed, M, H, Hkv, D, L, p):
    rng = np.random.default_rng(seed)
    ang = (np.arange(L)[:, None] * (10000.0 ** (-np.arange(D // 2) / (D // 2)))[None, :]).astype(np.float32)
    emb = np.concatenate([ang, ang], axis=-1)
    mask = np.ones((M, L), dtype=np.uint8)
    for m in range(M):
        mask[m, :min(m % 3, p)] = 0   # left padding; the new token's slot stays attendable
    return dict(q=rand_bits(rng, (M, H * D)), k=rand_bits(rng, (M, Hkv * D)), v=rand_bits(rng, (M, Hkv * D)),
                kc=rand_bits(rng, (M, Hkv, L, D)), vc=rand_bits(rng, (M, Hkv, L, D)),
                cos=o.f32_to_bf16_bits(np.cos(emb)), sin=o.f32_to_bf16_bits(np.sin(emb)), mask=mask, p=p,
                H=H, Hkv=Hkv, D=D, L=L, scaling=D ** -0.5)


@pytest.mark.parametrize("M,H,Hkv,D,L,p", [(2, 4, 4, 64, 40, 17), (3, 8, 2, 128, 64, 63), (1, 2, 1, 64, 8, 0)])
def test_rope_attn_matches_library_attention(M, H, Hkv, D, L, p):
    import torch.nn.functional as F
    from transformers.models.llama.modeling_llama import apply_rotary_pos_emb

    c = attn_case(100 + p, M, H, Hkv, D, L, p)
    out, kc, vc = d.rope_attn_decode(c["q"], c["k"], c["v"], c["kc"], c["vc"], c["cos"], c["sin"], c["mask"],
                                     p, H, Hkv, c["scaling"])
    q = bits_to_bf16(c["q"]).view(M, 1, H, D).transpose(1, 2)
    k = bits_to_bf16(c["k"]).view(M, 1, Hkv, D).transpose(1, 2)
    v = bits_to_bf16(c["v"]).view(M, 1, Hkv, D).transpose(1, 2)
    cos, sin = bits_to_bf16(c["cos"])[p][None, None], bits_to_bf16(c["sin"])[p][None, None]
    qe, ke = apply_rotary_pos_emb(q, k, cos, sin)
    keys, values = bits_to_bf16(c["kc"]).clone(), bits_to_bf16(c["vc"]).clone()
    keys[:, :, p:p + 1], values[:, :, p:p + 1] = ke, v          # what StaticLayer.update does
    assert (kc == bf16_to_bits(keys)).all() and (vc == bf16_to_bits(values)).all()
    allowed = torch.from_numpy(c["mask"].astype(bool))[:, None, None, :] & (torch.arange(L) <= p)[None, None, None, :]
    want = F.scaled_dot_product_attention(qe.float(), keys.float().repeat_interleave(H // Hkv, dim=1),
                                          values.float().repeat_interleave(H // Hkv, dim=1),
                                          attn_mask=allowed, scale=c["scaling"])
    want = want.transpose(1, 2).reshape(M, H * D).double().numpy()
    assert np.abs(out - want).max() <= 1e-5 * max(1.0, np.abs(want).max())


def test_rope_attn_closed_forms():
    M, H, D, L = 2, 2, 64, 16
    c = attn_case(7, M, H, H, D, L, 9)
    only = np.zeros((M, L), dtype=np.uint8)
    only[:, 4] = 1                                             # one slot may be attended: its value row comes back
    out, _, _ = d.rope_attn_decode(c["q"], c["k"], c["v"], c["kc"], c["vc"], c["cos"], c["sin"], only, 9, H, H, 0.125)
    want = o.bf16_bits_to_f32(c["vc"][:, :, 4, :]).reshape(M, H * D)
    assert np.abs(out - want).max() == 0
    zero_q = np.zeros_like(c["q"])                             # all scores equal: the mean of the value rows 0..p
    out, _, vc = d.rope_attn_decode(zero_q, c["k"], c["v"], c["kc"], c["vc"], c["cos"], c["sin"],
                                    np.ones((M, L), dtype=np.uint8), 9, H, H, 0.125)
    want = o.bf16_bits_to_f32(vc[:, :, :10, :]).astype(np.float64).mean(axis=2).reshape(M, H * D)
    assert np.abs(out - want).max() <= 1e-12
    assert (vc[:, :, 9, :].reshape(M, H * D) == c["v"]).all() and (vc[:, :, 10:, :] == c["vc"][:, :, 10:, :]).all()


@pytest.mark.parametrize("fp32", [True, False])
def test_lora_add_matches_the_wrapper_formula_in_torch(fp32):
    """``base(x) + lora_B(lora_A(x)) * scaling`` with torch modules on the CPU, in the two dtypes a
    PEFT wrapper runs its adapter in."""
    from torch import nn

    rng = np.random.default_rng(3 + fp32)
    M, K, N, r, scaling = 5, 512, 96, 16, 2.0
    x, y = rand_bits(rng, (M, K)), rand_bits(rng, (M, N), 2.0)
    dtype = torch.float32 if fp32 else torch.bfloat16
    torch.manual_seed(int(fp32))
    lora_a, lora_b = nn.Linear(K, r, bias=False).to(dtype), nn.Linear(r, N, bias=False).to(dtype)
    with torch.no_grad():
        lora_b.weight.normal_(0, 0.05)
        result, xt = bits_to_bf16(y), bits_to_bf16(x)
        want = (result + lora_b(lora_a(xt.to(dtype))) * scaling).to(torch.bfloat16)
    got = d.lora_add(y, x, lora_a.weight.detach().float().numpy(), lora_b.weight.detach().float().numpy(), scaling, fp32)
    assert within_one_step_of(got, bf16_to_bits(want), y) < 0.02   # summation order inside the library products


def test_lora_add_closed_forms():
    rng = np.random.default_rng(9)
    M, K, N, r = 3, 64, 24, 8
    x, y = rand_bits(rng, (M, K)), rand_bits(rng, (M, N))
    A, B = rng.standard_normal((r, K)).astype(np.float32), np.zeros((N, r), dtype=np.float32)
    assert (d.lora_add(y, x, A, B, 2.0, True) == y).all()          # a fresh adapter (B = 0) changes nothing
    # rank-one adapter picking x[:, 0] into column 5: y[:, 5] + 2 * x[:, 0], one rounding
    A[:] = 0
    A[0, 0] = 1.0
    B[5, 0] = 1.0
    got = d.lora_add(y, x, A, B, 2.0, True)
    want = y.copy()
    want[:, 5] = o.f32_to_bf16_bits(o.bf16_bits_to_f32(y[:, 5]) + 2.0 * o.bf16_bits_to_f32(x[:, 0]))
    assert (got == want).all()
