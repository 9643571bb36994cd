"""Head + sampling tail in one launch (``vrl_int4_head_sample_bf16``) against the oracle (MI355X).

The fused launch must (a) produce the logits of the head linear (checked through ``logits_out`` against
the GEMV oracle and, bit for bit, against the plan-free launch it shares its tile code with) and (b) draw
and score exactly as ``oracle.cfg_sample`` does from those logits: the tokens equal unless the oracle's own
ratios show a near-tie, the log-probabilities within one bf16 step.
"""

import numpy as np
import pytest
import torch

from oracle import int4_oracle as o
from tests._util import assert_gemv_close, bf16_to_bits, bits_to_bf16, to_device
from tests.test_cfg_sample import check_against_oracle

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def ops_mod():
    from visionrl_amd import ops
    return ops


def make_head(seed, B, K, V, G, spread=24.0):
    """Operands of a head over 2B rows; the activations are scaled so that the logits spread like a
    trained head's (a flat distribution would make every draw a near-tie of thousands of entries)."""
    ops = o.make_operands(seed, 2 * B, K, V, G)
    x = o.bf16_bits_to_f32(ops["x_bits"]) * np.float32(spread / np.sqrt(K))
    ops["x_bits"] = o.f32_to_bf16_bits(x)
    rng = np.random.default_rng(seed + 1)
    nb = o.f32_to_bf16_bits(rng.exponential(1.0, size=(B, V)).astype(np.float32))
    nb[nb == 0] = 1
    return ops, nb


@pytest.mark.parametrize("B,K,V,G,w,T", [
    (1, 2048, 16384, 128, 5.0, 1.0),      # Janus-Pro-1B head, one image: 2 rows, one tile per workgroup
    (16, 2048, 16384, 128, 5.0, 1.0),     # the rollout batch: 32 rows, two row blocks per tile
    (3, 2048, 16384, 128, 1.5, 0.7),
    (8, 2048, 16384, 128, 5.0, 1.0),      # 16 rows: one full row block
    (9, 2048, 4096, 128, 7.5, 0.9),       # 18 rows: conditional rows straddle the two row blocks
    (1, 4096, 16384, 128, 5.0, 1.0),      # 7B-class head
    (8, 4096, 16384, 128, 5.0, 1.3),
    (5, 512, 1024, 64, 3.0, 1.0),
    (2, 1024, 48, 32, 0.0, 2.0),
])
def test_head_sample_matches_the_oracle(ops_mod, B, K, V, G, w, T):
    print(f"[case] head_sample B={B} K={K} V={V} G={G} w={w} T={T}", flush=True)
    ops, nb = make_head(700 + B + K + V, B, K, V, G)
    d = to_device(ops, DEV)
    pw = ops_mod.int4_prepack(d["qweight"], d["scales"], d["qzeros"], G)
    assert ops_mod.head_sample_supported(2 * B, pw)
    noise = bits_to_bf16(nb, DEV)
    logits = torch.empty((2 * B, V), dtype=torch.bfloat16, device=DEV)
    ws = ops_mod.head_sample_workspace(B, V, DEV)
    sampled, logprob = ops_mod.head_sample(d["x"], pw, w, T, noise=noise, logits_out=logits, workspace=ws)
    torch.cuda.synchronize()
    assert sampled.dtype == torch.int64 and logprob.dtype == torch.float32 and sampled.shape == (B,)
    lb = bf16_to_bits(logits)
    assert_gemv_close(lb, ops, G, f"head_sample logits B{B} K{K} V{V}")
    (plain,) = ops_mod.DirectGemv([(d["x"], pw, False)]).launch() if 2 * B <= 16 else (None,)
    if plain is not None:
        torch.cuda.synchronize()
        assert torch.equal(plain, logits)                              # the same tile code, the same sums
    exact = check_against_oracle(sampled, logprob, lb, nb, w, T)
    assert exact >= B - max(1, B // 8)
    # the launch of the tail alone over the same logits agrees (same arithmetic, other order of the sums)
    s2, lp2 = ops_mod.cfg_sample(logits, w, T, noise=noise)
    torch.cuda.synchronize()
    same = sampled == s2
    assert int(same.sum()) >= B - max(1, B // 8)
    assert torch.all((logprob[same] - lp2[same]).abs() <= 2.0 ** -7 * lp2[same].abs() + 1e-6)
    # without the logits output, and again over the same workspace: the same draw
    s3, lp3 = ops_mod.head_sample(d["x"], pw, w, T, noise=noise, workspace=ws)
    torch.cuda.synchronize()
    assert torch.equal(s3, sampled) and torch.equal(lp3, logprob)


def test_head_sample_repeats_over_one_workspace_and_follows_the_noise(ops_mod):
    """Calls back to back over one workspace, each with its own draws;
    constant noise samples the mode of the guided logits; a tiny draw wins."""
    print("[case] head_sample repeated calls and properties", flush=True)
    B, K, V, G = 16, 2048, 16384, 128
    ops, nb = make_head(811, B, K, V, G, spread=6.0)
    d = to_device(ops, DEV)
    pw = ops_mod.int4_prepack(d["qweight"], d["scales"], d["qzeros"], G)
    ws = ops_mod.head_sample_workspace(B, V, DEV)
    logits = torch.empty((2 * B, V), dtype=torch.bfloat16, device=DEV)
    rng = np.random.default_rng(5)
    runs = []
    for _ in range(4):                                                 # enqueued back to back, checked afterwards
        n = o.f32_to_bf16_bits(rng.exponential(1.0, size=(B, V)).astype(np.float32))
        n[n == 0] = 1
        runs.append((n, ops_mod.head_sample(d["x"], pw, 5.0, 1.0, noise=bits_to_bf16(n, DEV), logits_out=logits,
                                            workspace=ws)))
    torch.cuda.synchronize()
    lb = bf16_to_bits(logits)
    for n, (s, lp) in runs:
        assert check_against_oracle(s, lp, lb, n, 5.0, 1.0) >= B - 2
    ones = torch.ones((B, V), dtype=torch.bfloat16, device=DEV)
    s, lp = ops_mod.head_sample(d["x"], pw, 0.0, 1.0, noise=ones, workspace=ws)     # w = 0: guided = uncond
    assert torch.equal(s, torch.argmax(logits[B:].float(), dim=-1)) and bool((lp <= 0).all())
    tiny = ones.clone()
    tiny[:, 4321] = 1e-30
    s, _ = ops_mod.head_sample(d["x"], pw, 5.0, 1.0, noise=tiny, workspace=ws)
    assert bool((s == 4321).all())
    # seeded like torch.multinomial: the same stream as the two-launch path
    torch.manual_seed(99)
    a = ops_mod.head_sample(d["x"], pw, 5.0, 1.0, workspace=ws)
    torch.manual_seed(99)
    b = ops_mod.cfg_sample(logits, 5.0, 1.0)
    torch.cuda.synchronize()
    assert int((a[0] == b[0]).sum()) >= B - 1


def test_head_sample_inside_a_graph_equals_eager(ops_mod):
    """Recorded and replayed with eager work and synchronisations between the replays: every replay
    equals the eager call on the same inputs."""
    print("[case] head_sample graph replay", flush=True)
    B, K, V, G = 2, 2048, 16384, 128
    ops, nb = make_head(821, B, K, V, G)
    d = to_device(ops, DEV)
    pw = ops_mod.int4_prepack(d["qweight"], d["scales"], d["qzeros"], G)
    ws = ops_mod.head_sample_workspace(B, V, DEV)
    x, noise = d["x"].clone(), bits_to_bf16(nb, DEV)
    ops_mod.head_sample(x, pw, 5.0, 1.0, noise=noise, workspace=ws)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        out = ops_mod.head_sample(x, pw, 5.0, 1.0, noise=noise, workspace=ws)
    gen = torch.Generator(device=DEV).manual_seed(3)
    for _ in range(4):
        x.copy_((torch.randn((2 * B, K), generator=gen, device=DEV) * 0.5).to(torch.bfloat16))
        noise.exponential_(1.0, generator=gen)
        want = ops_mod.head_sample(x, pw, 5.0, 1.0, noise=noise, workspace=ws)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out[0], want[0]) and torch.equal(out[1], want[1])


def test_head_sample_refuses_what_it_does_not_take(ops_mod):
    ops, nb = make_head(831, 1, 512, 64, 128)
    d = to_device(ops, DEV)
    pw = ops_mod.int4_prepack(d["qweight"], d["scales"], d["qzeros"], 128)
    with pytest.raises(ValueError):
        ops_mod.head_sample(d["x"][:1], pw, 1.0, 1.0)                  # an odd number of rows
    with pytest.raises(ValueError):
        ops_mod.head_sample(d["x"], pw, 1.0, 0.0)
    with pytest.raises(ValueError):
        ops_mod.head_sample(torch.zeros((34, 512), dtype=torch.bfloat16, device=DEV), pw, 1.0, 1.0)   # B = 17
    with pytest.raises(ValueError):
        ops_mod.head_sample(d["x"], pw, 1.0, 1.0, workspace=torch.zeros(256, dtype=torch.uint8, device=DEV))
    big = o.make_operands(832, 2, 4096, 64, 128)
    db = to_device(big, DEV)
    wide = ops_mod.int4_prepack(db["qweight"], db["scales"], db["qzeros"], 128)
    assert not ops_mod.head_sample_supported(32, wide) and ops_mod.head_sample_supported(16, wide)


@pytest.mark.parametrize("B,K,V", [(1, 2048, 16384), (16, 2048, 16384), (5, 1024, 4096)])
def test_head_sample_with_bias_bookkeeping_and_next_embeddings(ops_mod, B, K, V):
    """``vrl_int4_head_sample_ex_bf16``: the biased logits are the plain launch's plus the bias with the module's
    two roundings; the draw over them is the oracle's; token and log-probability land at the device-side
    position of the step's buffers, position and slot move on by one, and rows b and B + b of the next input
    are the table's row of the sampled token.  Two calls in a row over one workspace."""
    print(f"[case] head_sample extras B={B} K={K} V={V}", flush=True)
    G, w, T, H, L = 128, 5.0, 1.0, 256, 40
    ops, nb = make_head(900 + B + K, B, K, V, G)
    d = to_device(ops, DEV)
    pw = ops_mod.int4_prepack(d["qweight"], d["scales"], d["qzeros"], G)
    rng = np.random.default_rng(B)
    bias_bits = o.f32_to_bf16_bits(rng.normal(0.0, 2.0, size=V).astype(np.float32))
    bias = bits_to_bf16(bias_bits, DEV)
    table = torch.randn((V, H), device=DEV).to(torch.bfloat16)
    nxt = torch.zeros((2 * B, 1, H), dtype=torch.bfloat16, device=DEV)
    tokens = torch.full((B, L), -1, dtype=torch.int64, device=DEV)
    lps = torch.full((B, L), 7.0, dtype=torch.float32, device=DEV)
    position = torch.tensor([17], dtype=torch.int64, device=DEV)
    slot = torch.tensor([300], dtype=torch.int64, device=DEV)
    ws = ops_mod.head_sample_workspace(B, V, DEV)
    plain = torch.empty((2 * B, V), dtype=torch.bfloat16, device=DEV)
    ops_mod.head_sample(d["x"], pw, w, T, noise=bits_to_bf16(nb, DEV), logits_out=plain, workspace=ws)
    logits = torch.empty_like(plain)
    for call in range(2):
        n = o.f32_to_bf16_bits(rng.exponential(1.0, size=(B, V)).astype(np.float32))
        n[n == 0] = 1
        sampled, lp = ops_mod.head_sample(d["x"], pw, w, T, noise=bits_to_bf16(n, DEV), logits_out=logits,
                                          workspace=ws, bias=bias, bookkeeping=(tokens, lps, position, slot),
                                          embedding=(table, nxt))
        torch.cuda.synchronize()
        assert torch.equal(logits, plain + bias)                  # bf16(bf16(x . W^T) + bias), as the module adds it
        assert check_against_oracle(sampled, lp, bf16_to_bits(logits), n, w, T) >= B - max(1, B // 8)
        assert int(position) == 18 + call and int(slot) == 301 + call
        assert torch.equal(tokens[:, 17 + call], sampled) and torch.equal(lps[:, 17 + call], lp)
        assert torch.equal(nxt[:B, 0], table[sampled]) and torch.equal(nxt[B:, 0], table[sampled])
    assert int((tokens != -1).sum()) == 2 * B and int((lps != 7.0).sum()) == 2 * B
    # without a slot the cache counter stays; a position past the buffers writes nothing
    position.fill_(L)
    ops_mod.head_sample(d["x"], pw, w, T, workspace=ws, bookkeeping=(tokens, lps, position, None))
    torch.cuda.synchronize()
    assert int(position) == L + 1 and int(slot) == 302 and int((tokens != -1).sum()) == 2 * B


@pytest.mark.parametrize("M,K,N,G,norm", [(2, 2048, 2048, 128, False), (2, 2048, 2048, 128, True),
                                          (32, 2048, 2048, 128, True), (8, 4096, 4096, 128, True),
                                          (5, 1024, 1536, 64, False), (32, 5632, 2048, 128, False),
                                          (16, 2048, 2048, 128, False), (2, 5632, 2048, 128, False),
                                          (32, 11008, 4096, 128, False), (32, 4096, 4096, 128, False),
                                          (24, 3072, 2048, 64, False), (6, 2048, 2048, 128, False),
                                          (12, 5632, 2048, 128, False)])
def test_linear_with_bias_and_gelu_in_one_launch(ops_mod, M, K, N, G, norm):
    """``vrl_int4_gemv_prepacked_epilogue_bf16`` (the front of a two-layer head): bit for bit what the plain
    launch followed by the tensor ops gives (bias added to the bf16 output, exact GELU in fp32 on the bf16
    value), and the linear itself against the oracle; with the trunk's last norm folded in, against the
    normalising launch."""
    print(f"[case] epilogue launch M={M} K={K} N={N} G={G} norm={norm}", flush=True)
    ops = o.make_operands(1200 + M + K + N, M, K, N, G)
    d = to_device(ops, DEV)
    pw = ops_mod.int4_prepack(d["qweight"], d["scales"], d["qzeros"], G)
    gen = torch.Generator(device=DEV).manual_seed(M + K)
    bias = torch.randn(N, generator=gen, device=DEV).to(torch.bfloat16)
    norm_args = None
    if norm:
        res = torch.randn((M, K), generator=gen, device=DEV).to(torch.bfloat16)
        nw = (1.0 + 0.1 * torch.randn(K, generator=gen, device=DEV)).to(torch.bfloat16)
        norm_args = (res, nw, 1e-6)
        (base,) = ops_mod.DirectGemv([(d["x"], pw, False)], norm=(res, nw, 1e-6, None)).launch()
    else:
        # the linear alone through the same launch form (a bias of zeros changes no bit); the plain launch of 17 to
        # 32 rows may split K differently
        base = ops_mod.EpilogueGemv(d["x"], pw, torch.zeros_like(bias)).launch().clone()
        torch.cuda.synchronize()
        assert_gemv_close(bf16_to_bits(base), ops, G, f"epilogue base M{M} K{K} N{N}")
        if M <= 16:
            (plain,) = ops_mod.DirectGemv([(d["x"], pw, False)]).launch()
            torch.cuda.synchronize()
            assert torch.equal(base, plain)
    for b, gelu in ((bias, True), (bias, False), (None, True)):
        got = ops_mod.EpilogueGemv(d["x"], pw, b, gelu=gelu, norm=norm_args).launch()
        want = base if b is None else base + b
        want = torch.nn.functional.gelu(want) if gelu else want
        torch.cuda.synchronize()
        assert torch.equal(got, want), (b is not None, gelu, (got.float() - want.float()).abs().max().item())
    # the sublayer's output joining a residual stream in the same launch (o_proj, down_proj of a decoder layer):
    # bf16(residual + bf16(x . W^T)); also into the residual's own memory
    stream = torch.randn((M, N), generator=gen, device=DEV).to(torch.bfloat16)
    got = ops_mod.EpilogueGemv(d["x"], pw, residual=stream, norm=norm_args).launch()
    torch.cuda.synchronize()
    assert torch.equal(got, stream + base)
    got = ops_mod.EpilogueGemv(d["x"], pw, bias, gelu=True, residual=stream, norm=norm_args).launch()
    torch.cuda.synchronize()
    assert torch.equal(got, stream + torch.nn.functional.gelu(base + bias))
    in_place = stream.clone()
    ops_mod.EpilogueGemv(d["x"], pw, residual=in_place, out=in_place, norm=norm_args).launch()
    torch.cuda.synchronize()
    assert torch.equal(in_place, stream + base)
    with pytest.raises(ValueError):
        ops_mod.EpilogueGemv(d["x"], pw, bias[:-1].contiguous())
    with pytest.raises(ValueError):
        ops_mod.EpilogueGemv(d["x"], pw, residual=stream[:, :-8].contiguous())
