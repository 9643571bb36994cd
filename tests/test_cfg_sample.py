"""Decode-step tail (CFG combine, softmax, one draw, its log-probability): oracle pins and GPU parity."""
import numpy as np
import pytest
import torch

from oracle import int4_oracle as o
from tests._util import bits_to_bf16

DEV = "cuda:0"


def make_logits(seed, B, V, spread=3.0):
    rng = np.random.default_rng(seed)
    logits = (rng.standard_normal((2 * B, V)) * spread).astype(np.float32)
    noise = rng.exponential(1.0, size=(B, V)).astype(np.float32)
    nb = o.f32_to_bf16_bits(noise)
    nb[nb == 0] = 1                          # strictly positive, as torch's exponential_ guarantees
    return o.f32_to_bf16_bits(logits), nb


# ------------------------------------------------------------------ oracle pinned by what the mathematics fixes
def test_oracle_against_closed_forms():
    lb, nb = make_logits(1, 3, 257)
    # all draws equal: the sample is the most probable token, i.e. the first maximum of guided
    ones = np.full_like(nb, 0x3F80)
    s, lp, probs, _ = o.cfg_sample(lb, ones, 1.0, 1.0)
    c = o.bf16_bits_to_f32(lb[:3]); u = o.bf16_bits_to_f32(lb[3:])
    # w = 1, T = 1: guided = bf16(u + bf16(c - u)), evaluated here independently in float64 with explicit roundings
    rb = lambda v: o.bf16_bits_to_f32(o.f32_to_bf16_bits(np.asarray(v, dtype=np.float64).astype(np.float32))).astype(np.float64)
    guided = rb(u.astype(np.float64) + rb(c.astype(np.float64) - u))
    assert (s == np.argmax(guided, axis=1)).all()
    # probabilities are a bf16 rounding of a distribution: sum within V half-ulps of 1
    assert np.all(np.abs(probs.sum(axis=1) - 1.0) < 257 * 2.0 ** -9)
    # log-probability of the sample against a float64 log-softmax of cond
    ref = c.astype(np.float64) - np.log(np.exp(c.astype(np.float64) - c.max(1, keepdims=True)).sum(1, keepdims=True)) \
        - c.max(1, keepdims=True)
    want = ref[np.arange(3), s]
    assert np.all(np.abs(lp - want) <= np.maximum(o.bf16_ulp(want), 2.0 ** -8))
    # w = 0: the draw ignores cond; a wrong sign or swapped operand in the combine shows here
    s0, _, p0, _ = o.cfg_sample(lb, ones, 0.0, 1.0)
    assert (s0 == np.argmax(u, axis=1)).all()
    # temperature: T -> small sharpens, the top probability grows
    _, _, p_cold, _ = o.cfg_sample(lb, ones, 0.0, 0.25)
    assert (p_cold.max(1) >= p0.max(1)).all()


def test_oracle_draw_follows_the_noise():
    """argmax(p / q): dividing one token's draw by a large factor makes it the sample."""
    lb, nb = make_logits(2, 2, 64, spread=0.5)
    for tok in (0, 17, 63):
        n2 = nb.copy()
        n2[:, tok] = o.f32_to_bf16_bits(np.full(2, 1e-6, dtype=np.float32))
        s, _, _, _ = o.cfg_sample(lb, n2, 3.0, 1.0)
        assert (s == tok).all()


def test_oracle_matches_the_torch_ops_it_restates():
    """The same tensor ops as policy.py:686-693, run by torch on the CPU in bfloat16.

    Temperatures are powers of two here: dividing by them and multiplying by their reciprocal is
    the same arithmetic (torch's CPU kernel divides, its device kernel multiplies by fl(1/T), which
    is what the oracle restates; other temperatures are compared on the device)."""
    import torch.nn.functional as F
    lb, nb = make_logits(3, 4, 512)
    logits = bits_to_bf16(lb)
    q = bits_to_bf16(nb)
    for w, T in ((5.0, 1.0), (1.5, 0.5), (0.0, 2.0)):
        cond, uncond = logits.chunk(2, dim=0)
        guided = uncond + w * (cond - uncond)
        probs = F.softmax(guided / T, dim=-1)
        sampled = torch.argmax(probs / q, dim=-1)                 # what multinomial(probs, 1) computes from q
        lp = F.log_softmax(cond / T, dim=-1).gather(-1, sampled.unsqueeze(-1)).squeeze(-1)
        s, l, p, ratio = o.cfg_sample(lb, nb, w, T)
        # probabilities within one bf16 ulp (torch's CPU kernels may divide by T instead of multiplying by 1/T
        # and sum in another order); the draw equal, or a near-tie of the oracle's own ratios
        assert np.all(np.abs(p - probs.float().numpy()) <= o.bf16_ulp(p.astype(np.float64)) + 1e-30)
        ts = sampled.numpy()
        for b in range(4):
            assert s[b] == ts[b] or ratio[b, ts[b]] >= ratio[b].max() * (1 - 2.0 ** -6), (w, T, b)
        # log-probability: one rounding away from the float64 log-softmax of the bf16 cond / T
        # (torch's CPU bf16 log_softmax rounds an intermediate and is coarser than its device kernel)
        del lp
        lp64 = F.log_softmax((cond / T).double(), dim=-1).numpy()[np.arange(4), s]
        assert np.all(np.abs(l - lp64) <= o.bf16_ulp(lp64) + 1e-6)


# ------------------------------------------------------------------ GPU parity
@pytest.fixture(scope="module")
def ops_mod():
    from visionrl_amd import ops
    return ops


def check_against_oracle(sampled, logprob, lb, nb, w, T):
    s, l, _, ratio = o.cfg_sample(lb, nb, w, T)
    got_s, got_l = sampled.cpu().numpy(), logprob.cpu().numpy()
    exact = 0
    for b in range(len(s)):
        if got_s[b] == s[b]:
            exact += 1
            # same token: the log-probability is one bf16 value or its neighbour (fp32 sum order, exp)
            assert abs(got_l[b] - l[b]) <= o.bf16_ulp(np.float64(l[b])), (b, got_l[b], l[b])
        else:
            # another token only where the oracle itself sees a near-tie of probs / noise
            assert ratio[b, got_s[b]] >= ratio[b].max() * (1 - 2.0 ** -6), (b, got_s[b], s[b])
    return exact


@pytest.mark.gpu
@pytest.mark.parametrize("B,V,w,T", [(1, 16384, 5.0, 1.0), (16, 16384, 5.0, 1.0), (3, 1000, 1.5, 0.7),
                                     (2, 17, 0.0, 2.0), (5, 65536 + 24, 7.5, 0.9), (16, 16384, 1.0, 1.0),
                                     (2, 8192, 3.0, 1.0), (4, 8192 + 64, 5.0, 1.3)])
def test_cfg_sample_matches_oracle(ops_mod, B, V, w, T):
    print(f"[case] cfg_sample B={B} V={V} w={w} T={T}", flush=True)
    lb, nb = make_logits(40 + B + V, B, V)
    sampled, logprob = ops_mod.cfg_sample(bits_to_bf16(lb, DEV), w, T, noise=bits_to_bf16(nb, DEV))
    torch.cuda.synchronize()
    assert sampled.dtype == torch.int64 and logprob.dtype == torch.float32
    exact = check_against_oracle(sampled, logprob, lb, nb, w, T)
    assert exact >= B - max(1, B // 8)


@pytest.mark.gpu
def test_cfg_sample_draws_like_torch_multinomial(ops_mod):
    """Seeded: the fused launch samples the tokens the reference's tensor ops sample (policy.py:686-693),
    because it draws its noise with the call torch.multinomial makes."""
    import torch.nn.functional as F
    print("[case] cfg_sample vs torch ops on the device", flush=True)
    B, V = 16, 16384
    lb, _ = make_logits(77, B, V)
    logits = bits_to_bf16(lb, DEV)
    same = 0
    for seed, (w, T) in enumerate(((5.0, 1.0), (5.0, 1.0), (1.5, 0.7), (7.5, 0.9))):
        torch.manual_seed(1234 + seed)
        cond, uncond = logits.chunk(2, dim=0)
        guided = uncond + w * (cond - uncond)
        probs = F.softmax(guided / T, dim=-1)
        want = torch.multinomial(probs, num_samples=1).squeeze(-1)
        want_lp = F.log_softmax(cond / T, dim=-1).gather(-1, want.unsqueeze(-1)).squeeze(-1)
        torch.manual_seed(1234 + seed)
        got, got_lp = ops_mod.cfg_sample(logits, w, T)
        torch.cuda.synchronize()
        eq = (got == want)
        same += int(eq.sum())
        assert torch.all((got_lp[eq] - want_lp.float()[eq]).abs() <= 2.0 ** -7 * want_lp.float()[eq].abs() + 1e-6)
    assert same >= 4 * B - 2          # near-ties of probs / noise may resolve differently, nothing else


@pytest.mark.gpu
def test_cfg_sample_properties_at_full_size(ops_mod):
    """Size-independent facts at the rollout shape: constant noise samples the mode; a tiny draw wins."""
    print("[case] cfg_sample properties", flush=True)
    B, V = 16, 16384
    lb, nb = make_logits(91, B, V, spread=0.25)                     # flat enough that no probability rounds to zero
    logits = bits_to_bf16(lb, DEV)
    ones = torch.ones((B, V), dtype=torch.bfloat16, device=DEV)
    s, lp = ops_mod.cfg_sample(logits, 0.0, 1.0, noise=ones)       # w = 0: guided = uncond
    assert torch.equal(s, torch.argmax(logits[B:].float(), dim=-1))
    assert bool((lp <= 0).all())
    tiny = ones.clone()
    tiny[:, 4321] = 1e-30
    s, _ = ops_mod.cfg_sample(logits, 5.0, 1.0, noise=tiny)
    assert bool((s == 4321).all())
    with pytest.raises(ValueError):
        ops_mod.cfg_sample(logits[:3], 1.0, 1.0)
    with pytest.raises(ValueError):
        ops_mod.cfg_sample(logits, 1.0, 0.0)
