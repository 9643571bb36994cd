"""The decode-step kernels between the linears against their oracle (and against the library
modules they stand for, run on the device)."""

import numpy as np
import pytest
import torch

from oracle import decode_oracle as d
from oracle import int4_oracle as o
from tests._util import bf16_to_bits, bits_to_bf16
from tests.test_decode_oracle import attn_case, rand_bits, ulp_distance, within_one_step_of

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


@pytest.fixture(scope="module")
def ops_mod():
    from visionrl_amd import ops
    return ops


def say(*what):
    print("decode layer:", *what, flush=True)


@pytest.mark.parametrize("M,K,with_residual", [(1, 2048, False), (2, 2048, True), (32, 2048, True), (3, 4096, True),
                                               (5, 264, True), (2, 16384, False), (7, 3072, True)])
def test_add_rmsnorm_parity(ops_mod, M, K, with_residual):
    say("add_rmsnorm", M, K, with_residual)
    rng = np.random.default_rng(31 * K + M)
    x, res, w = rand_bits(rng, (M, K)), rand_bits(rng, (M, K), 4.0), rand_bits(rng, (K,), 0.5)
    h_want, y_want = d.add_rmsnorm(x, res if with_residual else None, w, 1e-6)
    xt, rt, wt = bits_to_bf16(x, DEV), bits_to_bf16(res, DEV), bits_to_bf16(w, DEV)
    h, y = ops_mod.add_rmsnorm(xt, wt, 1e-6, rt if with_residual else None)
    torch.cuda.synchronize()
    assert (bf16_to_bits(h) == h_want).all()
    dist = ulp_distance(bf16_to_bits(y), y_want)
    assert dist.max() <= 1 and (dist > 0).mean() < 2e-3, (dist.max(), (dist > 0).mean())
    if with_residual:   # in place: h over the residual stream
        h2, y2 = ops_mod.add_rmsnorm(xt, wt, 1e-6, rt, h_out=rt)
        torch.cuda.synchronize()
        assert h2 is rt and torch.equal(h2, h) and torch.equal(y2, y)


def test_add_rmsnorm_equals_the_library_module_on_the_device(ops_mod):
    from transformers.models.llama.modeling_llama import LlamaRMSNorm

    say("add_rmsnorm vs LlamaRMSNorm")
    torch.manual_seed(0)
    norm = LlamaRMSNorm(2048, eps=1e-6).to(torch.bfloat16).to(DEV)
    with torch.no_grad():
        norm.weight.normal_(1.0, 0.2)
        x = torch.randn(32, 2048, device=DEV).to(torch.bfloat16)
        res = (torch.randn(32, 2048, device=DEV) * 5).to(torch.bfloat16)
        want_h = res + x
        want = norm(want_h)
    h, y = ops_mod.add_rmsnorm(x, norm.weight.data, 1e-6, res)
    torch.cuda.synchronize()
    assert torch.equal(h, want_h)
    dist = ulp_distance(bf16_to_bits(y), bf16_to_bits(want))
    assert dist.max() <= 1 and (dist > 0).mean() < 2e-3


def run_attn(ops_mod, c):
    t = {k: (bits_to_bf16(c[k], DEV) if k in ("q", "k", "v", "kc", "vc", "cos", "sin") else None) for k in c}
    mask = torch.from_numpy(c["mask"]).to(DEV)
    pos = torch.tensor([c["p"]], dtype=torch.int64, device=DEV)
    out = ops_mod.rope_attn_decode(t["q"], t["k"], t["v"], t["kc"], t["vc"], t["cos"], t["sin"], mask, pos,
                                   c["scaling"])
    torch.cuda.synchronize()
    return out, t["kc"], t["vc"]


ATTN_CASES = [
    # M, H, Hkv, D, L, p
    (2, 16, 16, 128, 640, 37), (2, 16, 16, 128, 640, 639), (32, 16, 16, 128, 128, 100), (3, 4, 4, 64, 64, 0),
    (3, 4, 4, 64, 64, 1), (2, 8, 2, 128, 96, 15), (2, 8, 2, 128, 96, 16), (2, 8, 2, 128, 96, 17), (1, 6, 3, 64, 48, 47),
    (2, 4, 1, 64, 8192, 5000),
]


@pytest.mark.parametrize("M,H,Hkv,D,L,p", ATTN_CASES)
def test_rope_attn_decode_parity(ops_mod, M, H, Hkv, D, L, p):
    say("rope_attn", M, H, Hkv, D, L, p)
    c = attn_case(1000 + p + L, M, H, Hkv, D, L, p)
    want, kc_want, vc_want = d.rope_attn_decode(c["q"], c["k"], c["v"], c["kc"], c["vc"], c["cos"], c["sin"],
                                                c["mask"], p, H, Hkv, c["scaling"])
    out, kc, vc = run_attn(ops_mod, c)
    # cache: slot p holds the rotated key and the value bit for bit, nothing else moved
    assert (bf16_to_bits(kc) == kc_want).all() and (bf16_to_bits(vc) == vc_want).all()
    got = o.bf16_bits_to_f32(bf16_to_bits(out)).astype(np.float64)
    # fp32 scores and accumulation, one bf16 rounding of the result
    tol = 0.51 * o.bf16_ulp(want.astype(np.float32)) + 2e-5 * np.abs(want).max()
    assert (np.abs(got - want) <= tol).all(), np.abs(got - want).max()


SPLIT_CASES = [
    # M, H, Hkv, D, L, p: 8 workgroups per pair up to 32 pairs, 4 up to 64, 2 up to 128; ranges of multiples of 64
    # slots: empty ranges, one partly filled range, exact multiples, a long cache.  Below 512 cached slots the
    # launch leaves a pair to its first workgroup (no exchange): both sides of that line, and on it
    (2, 16, 16, 128, 896, 511), (2, 16, 16, 128, 896, 513), (2, 16, 16, 128, 896, 600), (4, 16, 16, 128, 640, 600),
    (8, 16, 16, 128, 640, 639), (3, 4, 2, 64, 1024, 577),
    # two workgroups per pair (65 to 128 pairs) divide a pair from 768 slots on
    (8, 16, 16, 128, 1024, 767), (8, 16, 16, 128, 1024, 768), (8, 16, 16, 128, 1024, 1000),
    (2, 16, 16, 128, 896, 0), (2, 16, 16, 128, 896, 1), (2, 16, 16, 128, 896, 63), (2, 16, 16, 128, 896, 64),
    (2, 16, 16, 128, 896, 65), (2, 16, 16, 128, 896, 330), (2, 16, 16, 128, 896, 512), (2, 16, 16, 128, 896, 830),
    (2, 16, 16, 128, 896, 895), (4, 16, 16, 128, 384, 300), (8, 16, 16, 128, 384, 383), (1, 6, 3, 64, 48, 47),
    (2, 8, 2, 128, 2048, 2000), (3, 4, 4, 64, 8192, 5000),
]


def run_attn_split(ops_mod, c, ws, out=None):
    t = {k: bits_to_bf16(c[k], DEV) for k in ("q", "k", "v", "kc", "vc", "cos", "sin")}
    mask = torch.from_numpy(c["mask"]).to(DEV)
    pos = torch.tensor([c["p"]], dtype=torch.int64, device=DEV)
    out = ops_mod.rope_attn_decode(t["q"], t["k"], t["v"], t["kc"], t["vc"], t["cos"], t["sin"], mask, pos,
                                   c["scaling"], split_workspace=ws, out=out)
    return out, t["kc"], t["vc"]


@pytest.mark.parametrize("M,H,Hkv,D,L,p", SPLIT_CASES)
def test_split_rope_attn_decode_parity(ops_mod, M, H, Hkv, D, L, p):
    """The slots of a (row, head) pair divided over several workgroups, merged by the last to finish:
    same oracle, same bound, same cache update as the one-workgroup form; counters back at zero."""
    say("rope_attn split", M, H, Hkv, D, L, p)
    c = attn_case(3000 + p + L, M, H, Hkv, D, L, p)
    want, kc_want, vc_want = d.rope_attn_decode(c["q"], c["k"], c["v"], c["kc"], c["vc"], c["cos"], c["sin"],
                                                c["mask"], p, H, Hkv, c["scaling"])
    ws = ops_mod.rope_attn_split_workspace(M, H, D, DEV)
    out, kc, vc = run_attn_split(ops_mod, c, ws)
    torch.cuda.synchronize()
    assert (bf16_to_bits(kc) == kc_want).all() and (bf16_to_bits(vc) == vc_want).all()
    got = o.bf16_bits_to_f32(bf16_to_bits(out)).astype(np.float64)
    tol = 0.51 * o.bf16_ulp(want.astype(np.float32)) + 2e-5 * np.abs(want).max()
    assert (np.abs(got - want) <= tol).all(), np.abs(got - want).max()
    assert int(ws[: M * H * 4].view(torch.int32).abs().sum()) == 0          # ready for the next launch
    # the one-workgroup launch over the same inputs: equal up to the order of the fp32 sums
    plain, _, _ = run_attn(ops_mod, c)
    fa, fb = out.float(), plain.float()
    assert bool(((fa - fb).abs() <= fb.abs() * 2.0 ** -7 + 4e-5 * fb.abs().max()).all())
    assert float((out != plain).float().mean()) < 0.02


def test_split_rope_attn_launches_share_one_workspace(ops_mod):
    """Forty launches back to back over one workspace, every one with other inputs, positions and masks,
    checked afterwards: a launch must read what its own workgroups wrote, never what an earlier launch
    left in the workspace or in a cache; masked slots and an all-masked row included."""
    say("rope_attn split, repeated launches")
    M, H, D, L = 2, 16, 128, 1280    # positions on both sides of the 512 slots from which a pair is divided
    ws = ops_mod.rope_attn_split_workspace(M, H, D, DEV)
    rng = np.random.default_rng(77)
    runs = []
    for i in range(40):
        p = int(rng.integers(0, L))
        c = attn_case(4000 + i, M, H, H, D, L, p)
        if i % 5 == 1:
            c["mask"][0, : max(1, p // 2)] = 0
        if i % 7 == 3:
            c["mask"][1, :] = 0
        runs.append((c, run_attn_split(ops_mod, c, ws)))                  # enqueued, not yet checked
    torch.cuda.synchronize()
    for c, (out, kc, vc) in runs:
        with np.errstate(invalid="ignore"):   # the oracle's softmax of a row with nothing attendable is NaN
            want, kc_want, vc_want = d.rope_attn_decode(c["q"], c["k"], c["v"], c["kc"], c["vc"], c["cos"], c["sin"],
                                                        c["mask"], c["p"], H, H, c["scaling"])
        assert (bf16_to_bits(kc) == kc_want).all() and (bf16_to_bits(vc) == vc_want).all()
        got = o.bf16_bits_to_f32(bf16_to_bits(out)).astype(np.float64)
        dead = ~c["mask"][:, : c["p"] + 1].any(axis=1)        # nothing attendable: the launch writes zeros
        assert (got[dead] == 0).all()
        want, got = want[~dead], got[~dead]
        tol = 0.51 * o.bf16_ulp(want.astype(np.float32)) + 2e-5 * np.abs(want).max()
        assert (np.abs(got - want) <= tol).all(), (c["p"], np.abs(got - want).max())


def test_split_rope_attn_tracks_the_one_workgroup_form_over_many_launches(ops_mod):
    """Three hundred launches of both forms over one set of buffers, the position walking through a long cache
    and the new token changing every time, results compared on the device: within one bf16 step of each other
    (or, where an output cancels to almost nothing, within the fp32 noise of its terms), and different at all in
    fewer than 2 % of the outputs (the forms differ in the order of their fp32 sums only); a state left over from an earlier launch
    or a merge that ran before a state had arrived would be off by far more."""
    say("rope_attn split vs one-workgroup form, 300 launches")
    M, H, D, L = 2, 16, 128, 896
    c = attn_case(4300, M, H, H, D, L, 0)
    t = {k: bits_to_bf16(c[k], DEV) for k in ("q", "k", "v", "kc", "vc", "cos", "sin")}
    kc2, vc2 = t["kc"].clone(), t["vc"].clone()
    mask = torch.from_numpy(c["mask"]).to(DEV)
    pos = torch.zeros(1, dtype=torch.int64, device=DEV)
    ws = ops_mod.rope_attn_split_workspace(M, H, D, DEV)
    gen = torch.Generator(device=DEV).manual_seed(11)
    outs = []
    for step in range(300):
        pos.fill_((step * 37) % L)
        for name in ("q", "k", "v"):
            t[name].copy_((torch.randn(t[name].shape, generator=gen, device=DEV) * 0.7).to(torch.bfloat16))
        a = ops_mod.rope_attn_decode(t["q"], t["k"], t["v"], t["kc"], t["vc"], t["cos"], t["sin"], mask, pos,
                                     c["scaling"], split_workspace=ws)
        b = ops_mod.rope_attn_decode(t["q"], t["k"], t["v"], kc2, vc2, t["cos"], t["sin"], mask, pos, c["scaling"])
        outs.append((a, b))
    torch.cuda.synchronize()
    assert torch.equal(t["kc"], kc2) and torch.equal(t["vc"], vc2)
    differing = 0.0
    for a, b in outs:
        fa, fb = a.float(), b.float()
        # one bf16 step of the value, or for outputs that cancel to almost nothing the fp32 noise of O(1) terms
        tol = fb.abs() * 2.0 ** -7 + 4e-5 * fb.abs().max()
        assert bool(((fa - fb).abs() <= tol).all()), float((fa - fb).abs().max())
        differing += float((a != b).float().mean())
    assert differing / len(outs) < 0.02, differing / len(outs)
    assert int(ws[: M * H * 4].view(torch.int32).abs().sum()) == 0


def test_split_rope_attn_in_a_graph_equals_eager(ops_mod):
    """Recorded once, replayed with eager launches and synchronisations between the replays, the position
    advancing as in a decode loop: every replay equals the eager launch bit for bit (the merge runs in
    index order whichever workgroup arrives last).  The position crosses the 512 slots from which the launch
    divides a pair: the one recorded launch serves both sides."""
    say("rope_attn split, graph replay")
    M, H, D, L = 2, 16, 128, 896
    c = attn_case(4100, M, H, H, D, L, 200)
    t = {k: bits_to_bf16(c[k], DEV) for k in ("q", "k", "v", "kc", "vc", "cos", "sin")}
    mask = torch.from_numpy(c["mask"]).to(DEV)
    pos = torch.tensor([200], dtype=torch.int64, device=DEV)
    ws, ws_eager = (ops_mod.rope_attn_split_workspace(M, H, D, DEV) for _ in range(2))
    out = torch.empty((M, H * D), dtype=torch.bfloat16, device=DEV)
    call = lambda kc, vc, w, o_: ops_mod.rope_attn_decode(t["q"], t["k"], t["v"], kc, vc, t["cos"], t["sin"], mask,
                                                           pos, c["scaling"], split_workspace=w, out=o_)
    kc_g, vc_g = t["kc"].clone(), t["vc"].clone()
    call(kc_g, vc_g, ws, out)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call(kc_g, vc_g, ws, out)
    gen = torch.Generator(device=DEV).manual_seed(9)
    kc_e, vc_e = kc_g.clone(), vc_g.clone()
    for step in range(6):
        pos.fill_(421 + 37 * step)     # 421 ... 606
        for name in ("q", "k", "v"):
            t[name].copy_((torch.randn(t[name].shape, generator=gen, device=DEV) * 0.7).to(torch.bfloat16))
        want = call(kc_e, vc_e, ws_eager, None)
        torch.cuda.synchronize()
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, want) and torch.equal(kc_g, kc_e) and torch.equal(vc_g, vc_e)


def test_split_rope_attn_refuses_what_it_does_not_take(ops_mod):
    c = attn_case(4200, 2, 4, 4, 64, 32, 5)
    t = [bits_to_bf16(c[n], DEV) for n in ("q", "k", "v", "kc", "vc", "cos", "sin")]
    mask = torch.from_numpy(c["mask"]).to(DEV)
    pos = torch.tensor([5], dtype=torch.int64, device=DEV)
    with pytest.raises(ValueError):
        ops_mod.rope_attn_decode(*t, mask, pos, 0.125, split_workspace=torch.zeros(64, dtype=torch.uint8, device=DEV))
    with pytest.raises(ValueError):
        ops_mod.rope_attn_decode(*t, mask, pos, 0.125,
                                 split_workspace=ops_mod.rope_attn_split_workspace(2, 4, 64, DEV).float())
    # more pairs than the split form is for: the same entry point runs the one-workgroup launch
    big = attn_case(4201, 16, 16, 16, 64, 32, 7)
    ws = ops_mod.rope_attn_split_workspace(16, 16, 64, DEV)
    out, _, _ = run_attn_split(ops_mod, big, ws)
    plain, _, _ = run_attn(ops_mod, big)
    assert torch.equal(out, plain)


@pytest.mark.parametrize("M,H,Hkv,D,L,split", [(6, 16, 16, 128, 640, False), (6, 16, 16, 128, 640, True),
                                                (32, 16, 16, 128, 384, False), (4, 8, 2, 64, 96, False)])
def test_rope_attn_with_one_position_per_row(ops_mod, M, H, Hkv, D, L, split):
    """``vrl_rope_attn_decode_rows_bf16``: every row at its own slot (a chunk whose rows advance at different
    times).  Row m of the launch equals, bit for bit, row m of the one-position launch at that row's slot over
    the same cache; a row whose position lies outside the cache is left alone; the oracle agrees row by row."""
    say("rope_attn, one position per row", M, H, Hkv, D, L, split)
    rng = np.random.default_rng(M + L)
    positions = rng.integers(0, L, size=M)
    positions[0], positions[-1] = L - 1, 0
    if split:
        positions[1] = 600        # long enough for several workgroups per pair
    c = attn_case(4700 + M, M, H, Hkv, D, L, 0)
    t = {k: bits_to_bf16(c[k], DEV) for k in ("q", "k", "v", "kc", "vc", "cos", "sin")}
    mask = torch.from_numpy(c["mask"]).to(DEV)
    ws = ops_mod.rope_attn_split_workspace(M, H, D, DEV) if split else None
    kc, vc = t["kc"].clone(), t["vc"].clone()
    pos = torch.from_numpy(positions.astype(np.int64)).to(DEV)
    out = ops_mod.rope_attn_decode(t["q"], t["k"], t["v"], kc, vc, t["cos"], t["sin"], mask, pos, c["scaling"],
                                   split_workspace=ws, per_row=True)
    torch.cuda.synchronize()
    for p in sorted(set(positions.tolist())):
        rows = np.nonzero(positions == p)[0]
        kc1, vc1 = t["kc"].clone(), t["vc"].clone()
        ws1 = ops_mod.rope_attn_split_workspace(M, H, D, DEV) if split else None
        one = ops_mod.rope_attn_decode(t["q"], t["k"], t["v"], kc1, vc1, t["cos"], t["sin"], mask,
                                       torch.tensor([p], dtype=torch.int64, device=DEV), c["scaling"],
                                       split_workspace=ws1)
        torch.cuda.synchronize()
        assert torch.equal(out[rows], one[rows]), p
        assert torch.equal(kc[rows], kc1[rows]) and torch.equal(vc[rows], vc1[rows]), p
        want, _, _ = d.rope_attn_decode(c["q"], c["k"], c["v"], c["kc"], c["vc"], c["cos"], c["sin"], c["mask"], int(p),
                                        H, Hkv, c["scaling"])
        got = o.bf16_bits_to_f32(bf16_to_bits(out)).astype(np.float64)[rows]
        tol = 0.51 * o.bf16_ulp(want[rows].astype(np.float32)) + 2e-5 * np.abs(want[rows]).max()
        assert (np.abs(got - want[rows]) <= tol).all(), p
    if split:
        assert int(ws[: M * H * 4].view(torch.int32).abs().sum()) == 0
    # a row outside the cache: nothing of it is written, the others as before
    pos2 = pos.clone()
    pos2[2] = L + 5
    kc2, vc2 = t["kc"].clone(), t["vc"].clone()
    out2 = torch.full_like(out, 7.0)
    ops_mod.rope_attn_decode(t["q"], t["k"], t["v"], kc2, vc2, t["cos"], t["sin"], mask, pos2, c["scaling"],
                             out=out2, split_workspace=ws, per_row=True)
    torch.cuda.synchronize()
    keep = [m for m in range(M) if m != 2]
    assert torch.equal(out2[keep], out[keep]) and bool((out2[2] == 7.0).all())
    assert torch.equal(kc2[2], t["kc"][2]) and torch.equal(vc2[2], t["vc"][2])
    with pytest.raises(ValueError):
        ops_mod.rope_attn_decode(t["q"], t["k"], t["v"], kc2, vc2, t["cos"], t["sin"], mask, pos2[:1], c["scaling"],
                                 per_row=True)


def test_rope_attn_masks_and_strided_inputs(ops_mod):
    say("rope_attn masks, fused qkv buffer")
    M, H, D, L, p = 2, 4, 64, 32, 20
    c = attn_case(5, M, H, H, D, L, p)
    c["mask"][:] = 0
    c["mask"][:, 4] = 1           # one slot allowed: the output is that slot's value row
    out, _, _ = run_attn(ops_mod, c)
    assert (bf16_to_bits(out) == c["vc"][:, :, 4, :].reshape(M, H * D)).all()
    c["mask"][:] = 0              # nothing allowed: zeros, not NaN
    out, _, _ = run_attn(ops_mod, c)
    assert (bf16_to_bits(out) & 0x7FFF == 0).all()
    # q, k, v as column blocks of one [M, 3*H*D] buffer (how a fused projection would hand them over)
    c = attn_case(6, M, H, H, D, L, p)
    want, _, _ = run_attn(ops_mod, c)
    qkv = torch.cat([bits_to_bf16(c[n], DEV) for n in ("q", "k", "v")], dim=1)
    q, k, v = qkv[:, :H * D], qkv[:, H * D:2 * H * D], qkv[:, 2 * H * D:]
    got = ops_mod.rope_attn_decode(q, k, v, bits_to_bf16(c["kc"], DEV), bits_to_bf16(c["vc"], DEV),
                                   bits_to_bf16(c["cos"], DEV), bits_to_bf16(c["sin"], DEV),
                                   torch.from_numpy(c["mask"]).to(DEV),
                                   torch.tensor([p], dtype=torch.int64, device=DEV), c["scaling"])
    torch.cuda.synchronize()
    assert torch.equal(got, want)


@pytest.mark.parametrize("M,H,Hkv,D,L,p", [(2, 16, 16, 128, 640, 0), (2, 16, 16, 128, 640, 1), (2, 16, 16, 128, 640, 37),
                                           (2, 16, 16, 128, 640, 127), (2, 16, 16, 128, 640, 128),
                                           (2, 16, 16, 128, 640, 129), (2, 16, 16, 128, 640, 600),
                                           (3, 4, 2, 64, 40, 33), (2, 8, 2, 128, 24, 5)])
def test_rope_attn_ignores_what_the_slots_past_the_position_hold(ops_mod, M, H, Hkv, D, L, p):
    """Slots at and past the row's position have not been written by this sequence: whatever bits they hold
    (infinities and NaNs included, which a weight of zero would not silence) the result and the slots
    themselves are what a cache of ordinary values there gives, for the one-workgroup and the split form."""
    say("rope_attn poisoned tail", M, H, Hkv, D, L, p)
    c = attn_case(7000 + p + L, M, H, Hkv, D, L, p)
    want, kc_want, vc_want = run_attn(ops_mod, c)
    poison = np.array([0x7FC0, 0x7F80, 0xFF80, 0xFFFF], dtype=np.uint16)
    bad = dict(c)
    bad["kc"], bad["vc"] = c["kc"].copy(), c["vc"].copy()
    tail = bad["kc"][:, :, p:, :]
    bad["kc"][:, :, p:, :] = poison[np.arange(tail.size).reshape(tail.shape) % 4]
    bad["vc"][:, :, p:, :] = poison[(np.arange(tail.size).reshape(tail.shape) + 1) % 4]
    bad["mask"] = np.zeros_like(c["mask"])         # nor does the mask past the position matter
    bad["mask"][:, :p + 1] = c["mask"][:, :p + 1]
    out, kc, vc = run_attn(ops_mod, bad)
    assert torch.equal(out, want)
    assert torch.equal(kc[:, :, :p + 1], kc_want[:, :, :p + 1]) and torch.equal(vc[:, :, :p + 1], vc_want[:, :, :p + 1])
    assert (bf16_to_bits(kc)[:, :, p + 1:] == bad["kc"][:, :, p + 1:]).all()
    ws = ops_mod.rope_attn_split_workspace(M, H, D, DEV)
    split_want, _, _ = run_attn_split(ops_mod, c, ws)
    split_out, _, _ = run_attn_split(ops_mod, bad, ws)
    torch.cuda.synchronize()
    assert torch.equal(split_out, split_want)


def test_position_outside_the_cache_is_a_no_op(ops_mod):
    say("rope_attn position out of range")
    c = attn_case(8, 2, 2, 2, 64, 16, 3)
    for bad in (-1, 16, 1 << 40):
        c["p"] = 3
        t_out = torch.full((2, 128), 7.0, dtype=torch.bfloat16, device=DEV)
        kc, vc = bits_to_bf16(c["kc"], DEV), bits_to_bf16(c["vc"], DEV)
        ops_mod.rope_attn_decode(bits_to_bf16(c["q"], DEV), bits_to_bf16(c["k"], DEV), bits_to_bf16(c["v"], DEV),
                                 kc, vc, bits_to_bf16(c["cos"], DEV), bits_to_bf16(c["sin"], DEV),
                                 torch.from_numpy(c["mask"]).to(DEV),
                                 torch.tensor([bad], dtype=torch.int64, device=DEV), c["scaling"], out=t_out)
        torch.cuda.synchronize()
        assert (t_out == 7.0).all() and (bf16_to_bits(kc) == c["kc"]).all() and (bf16_to_bits(vc) == c["vc"]).all()


def test_wrappers_reject_contract_violations(ops_mod):
    x = torch.zeros(2, 256, dtype=torch.bfloat16, device=DEV)
    w = torch.ones(256, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(ValueError):
        ops_mod.add_rmsnorm(x.float(), w, 1e-6)
    with pytest.raises(ValueError):
        ops_mod.add_rmsnorm(x, w[:128], 1e-6)
    with pytest.raises(ValueError):
        ops_mod.add_rmsnorm(x[:, :132].contiguous(), w[:132].contiguous(), 1e-6)   # K % 8
    c = attn_case(9, 2, 2, 2, 64, 16, 3)
    args = [bits_to_bf16(c[n], DEV) for n in ("q", "k", "v", "kc", "vc", "cos", "sin")]
    mask = torch.from_numpy(c["mask"]).to(DEV)
    pos = torch.tensor([3], dtype=torch.int64, device=DEV)
    with pytest.raises(ValueError):
        ops_mod.rope_attn_decode(*args, mask.long(), pos, 0.125)
    with pytest.raises(ValueError):
        ops_mod.rope_attn_decode(*args, mask, pos.int(), 0.125)
    with pytest.raises(ValueError):
        ops_mod.rope_attn_decode(args[0][:, :100], *args[1:], mask, pos, 0.125)


# ------------------------------------------------------------------ add + norm applied while the linears stage their input
NORM_FUSED_CASES = [
    # M, K, [N...], fused gate|up, residual
    (1, 2048, [2048, 2048, 2048], False, True), (2, 2048, [2048, 512, 512], False, True),
    (32, 2048, [2048, 2048, 2048], False, True), (2, 2048, [2 * 5632], True, True), (32, 2048, [2 * 704], True, True),
    (3, 4096, [256], False, False), (5, 640, [48, 80], False, True), (16, 1536, [64], False, True),
    (9, 2048, [100], False, False),
    # rows wider than 2048 with one wave per row (eight words per lane: the residual and the norm weight pass
    # through the registers in halves), incl. a K that is no multiple of 512 and the 7B-class shapes
    (16, 4096, [256, 128], False, True), (32, 4096, [2 * 1024], True, True), (5, 3072, [64], False, True),
    (7, 2560, [48], False, False), (32, 4096, [4096], False, True),
    # launches of many tiles take other workgroup shapes: wide rows with four waves per tile (two super-chunks each)
    # and four tiles per workgroup, fused records of 12+ rows with one tile, two slabs of rows, and rows of up to
    # 2048 values at 13 to 16 rows with eight waves per tile
    (8, 4096, [4096, 4096, 1024], False, True), (16, 4096, [4096, 4096], False, True),
    (4, 4096, [2 * 5632], True, True), (14, 4096, [2 * 5632], True, False), (24, 4096, [4096, 2048], False, True),
    (20, 4096, [2 * 5632], True, True), (14, 2048, [2048, 2048, 2048], False, True), (16, 2048, [2 * 5632], True, True),
]


@pytest.mark.parametrize("M,K,Ns,fused,with_residual", NORM_FUSED_CASES)
def test_norm_fused_launch_parity(ops_mod, M, K, Ns, fused, with_residual):
    from tests._util import assert_gate_up_close, assert_gemv_close, to_device

    say("norm-fused launch", M, K, Ns, fused, with_residual)
    G = 128
    rng = np.random.default_rng(7 * K + M)
    x, res, wn = rand_bits(rng, (M, K)), rand_bits(rng, (M, K), 4.0), rand_bits(rng, (K,), 0.5)
    h_want, xn = d.add_rmsnorm(x, res if with_residual else None, wn, 1e-6)
    xt, rt, wt = bits_to_bf16(x, DEV), bits_to_bf16(res, DEV), bits_to_bf16(wn, DEV)
    h_out = torch.zeros_like(xt)
    probs, checks = [], []
    for i, N in enumerate(Ns):
        ops = o.make_operands(4000 + i + N, M, K, N, G)
        ops["x_bits"] = xn                       # what the tiles must have multiplied
        dd = to_device(ops, DEV)
        probs.append((xt, ops_mod.int4_prepack(dd["qweight"], dd["scales"], dd["qzeros"], G), fused))
        checks.append(ops)
    outs = ops_mod.DirectGemv(probs, norm=(rt if with_residual else None, wt, 1e-6, h_out)).launch()
    torch.cuda.synchronize()
    assert (bf16_to_bits(h_out) == h_want).all()
    for y, ops in zip(outs, checks):
        if not fused:
            assert_gemv_close(bf16_to_bits(y), ops, G, "norm-fused")
            continue
        assert_gate_up_close(bf16_to_bits(y), ops, G, "norm-fused gate|up")
    # against the two-launch form on the device: same h, outputs within a rounding of the normalised row
    h2, normed = ops_mod.add_rmsnorm(xt, wt, 1e-6, rt if with_residual else None)
    two = ops_mod.DirectGemv([(normed, pw, f) for _, pw, f in probs]).launch()
    torch.cuda.synchronize()
    assert torch.equal(h2, h_out)
    for a, b in zip(outs, two):
        close = (a.float() - b.float()).abs() <= 2.0 ** -6 * b.float().abs() + 2.0 ** -7
        assert close.all() and (a != b).float().mean().item() < 0.02


def test_norm_fused_launch_rejects(ops_mod):
    G, M, K = 128, 2, 256
    ops = o.make_operands(1, M, K, 32, G)
    from tests._util import to_device
    dd = to_device(ops, DEV)
    pw = ops_mod.int4_prepack(dd["qweight"], dd["scales"], dd["qzeros"], G)
    x, w = dd["x"], torch.ones(K, dtype=torch.bfloat16, device=DEV)
    with pytest.raises(ValueError):
        ops_mod.DirectGemv([(x, pw, False), (x.clone(), pw, False)], norm=(None, w, 1e-6, None))   # two inputs
    with pytest.raises(ValueError):
        ops_mod.DirectGemv([(x, pw, False)], norm=(None, w[:128], 1e-6, None))
    with pytest.raises(ValueError):
        ops_mod.DirectGemv([(x, pw, False)], norm=(None, w, 1e-6, x)).launch()                     # h over x
    big = o.make_operands(2, 1, 8192, 16, G)
    db = to_device(big, DEV)
    pwb = ops_mod.int4_prepack(db["qweight"], db["scales"], db["qzeros"], G)
    with pytest.raises(ValueError):
        ops_mod.DirectGemv([(db["x"], pwb, False)],
                           norm=(None, torch.ones(8192, dtype=torch.bfloat16, device=DEV), 1e-6, None)).launch()


# ------------------------------------------------------------------ LoRA adapters over int4 projections
@pytest.mark.parametrize("M,K,shapes,fp32", [
    (2, 2048, [(2048, 32), (2048, 32), (2048, 32)], True), (32, 2048, [(2048, 32), (512, 32), (512, 32)], True),
    (2, 2048, [(2048, 32)], False), (7, 640, [(100, 8), (48, 16)], True), (32, 4096, [(4096, 64)], False),
    (1, 5632, [(2048, 64)], True), (9, 1024, [(96, 40), (64, 8)], False),
])
def test_lora_add_parity(ops_mod, M, K, shapes, fp32):
    say("lora add", M, K, shapes, fp32)
    rng = np.random.default_rng(K + M + len(shapes))
    dtype = torch.float32 if fp32 else torch.bfloat16
    x = rand_bits(rng, (M, K))
    xt = bits_to_bf16(x, DEV)
    adapters, checks = [], []
    for i, (N, r) in enumerate(shapes):
        A = torch.from_numpy((rng.standard_normal((r, K)) * K ** -0.5).astype(np.float32)).to(dtype)
        B = torch.from_numpy((rng.standard_normal((N, r)) * 0.1).astype(np.float32)).to(dtype)
        y = rand_bits(rng, (M, N), 2.0)
        yt = bits_to_bf16(y, DEV)
        scaling = 2.0 if i % 2 == 0 else 0.75
        adapters.append((A.to(DEV), B.to(DEV), scaling, yt))
        checks.append((y, A.float().numpy(), B.float().numpy(), scaling, yt))
    ops_mod.LoraAdd(xt, adapters).launch()
    torch.cuda.synchronize()
    for y, A, B, scaling, yt in checks:
        want = d.lora_add(y, x, A, B, scaling, fp32)
        assert within_one_step_of(bf16_to_bits(yt), want, y) < 0.02


def test_lora_add_sees_in_place_weight_updates_and_rejects_misuse(ops_mod):
    say("lora add: weight sync, contract")
    rng = np.random.default_rng(1)
    M, K, N, r = 2, 256, 64, 8
    x = rand_bits(rng, (M, K))
    xt = bits_to_bf16(x, DEV)
    A = torch.zeros(r, K, device=DEV)
    B = torch.zeros(N, r, device=DEV)
    y0 = rand_bits(rng, (M, N))
    yt = bits_to_bf16(y0, DEV)
    launch = ops_mod.LoraAdd(xt, [(A, B, 2.0, yt)])
    launch.launch()
    torch.cuda.synchronize()
    assert (bf16_to_bits(yt) == y0).all()                      # B = 0: nothing added
    A.copy_(torch.randn(r, K, device=DEV) * 0.1)               # what a LoRA weight sync does
    B.copy_(torch.randn(N, r, device=DEV) * 0.1)
    launch.launch()
    torch.cuda.synchronize()
    want = d.lora_add(y0, x, A.cpu().numpy(), B.cpu().numpy(), 2.0, True)
    within_one_step_of(bf16_to_bits(yt), want, y0)
    with pytest.raises(ValueError):
        ops_mod.LoraAdd(xt, [(A, B.to(torch.bfloat16), 2.0, yt)])       # mixed dtypes
    with pytest.raises(ValueError):
        ops_mod.LoraAdd(xt, [(A[:, :128].contiguous(), B, 2.0, yt)])    # A does not take x
    with pytest.raises(ValueError):
        ops_mod.LoraAdd(xt, [(A, B, 2.0, yt)] * 5)
    with pytest.raises(ValueError):
        ops_mod.LoraAdd(xt, [(A[:4].contiguous(), B[:, :4].contiguous(), 2.0, yt)]).launch()   # rank % 8
    with pytest.raises(ValueError):
        ops_mod.LoraAdd(xt, [(A, B, 2.0, yt), (A.to(torch.bfloat16), B.to(torch.bfloat16), 2.0, yt)])   # one type per launch


@pytest.mark.parametrize("M,H,Hkv,D,fp32,which", [(2, 16, 16, 128, True, "qkv"), (32, 16, 16, 128, True, "qkv"),
                                                   (3, 8, 2, 64, False, "qv"), (5, 4, 4, 64, True, "k")])
def test_attention_adds_the_qkv_adapters_itself(ops_mod, M, H, Hkv, D, fp32, which):
    """``rope_attn_decode(..., lora=group)`` against the two-launch form (up-projection onto q, k, v,
    then the plain attention): the appended cache rows and the output agree to a rounding of the
    adapter sums' order."""
    say("attention with adapters", M, H, Hkv, D, fp32, which)
    L, p, K, r = 96, 41, 256, 16
    c = attn_case(300 + M, M, H, Hkv, D, L, p)
    rng = np.random.default_rng(M + D)
    dtype = torch.float32 if fp32 else torch.bfloat16
    x = bits_to_bf16(rand_bits(rng, (M, K)), DEV)
    t = {n: bits_to_bf16(c[n], DEV) for n in ("q", "k", "v", "cos", "sin")}
    mask = torch.from_numpy(c["mask"]).to(DEV)
    pos = torch.tensor([p], dtype=torch.int64, device=DEV)

    def adapters(q, k, v):
        gen = torch.Generator().manual_seed(5)
        ads = []
        for name, y in (("q", q), ("k", k), ("v", v)):
            if name in which:
                A = (torch.randn(r, K, generator=gen) * K ** -0.5).to(dtype).to(DEV)
                B = (torch.randn(y.shape[1], r, generator=gen) * 0.2).to(dtype).to(DEV)
                ads.append((A, B, 2.0, y))
        return ads

    # two launches: y += up(down(x)), then attention
    q1, k1, v1 = t["q"].clone(), t["k"].clone(), t["v"].clone()
    kc1, vc1 = bits_to_bf16(c["kc"], DEV), bits_to_bf16(c["vc"], DEV)
    ops_mod.LoraAdd(x, adapters(q1, k1, v1)).launch()
    want = ops_mod.rope_attn_decode(q1, k1, v1, kc1, vc1, t["cos"], t["sin"], mask, pos, c["scaling"])
    # one: down only, the attention adds the rest
    q2, k2, v2 = t["q"].clone(), t["k"].clone(), t["v"].clone()
    kc2, vc2 = bits_to_bf16(c["kc"], DEV), bits_to_bf16(c["vc"], DEV)
    group = ops_mod.LoraAdd(x, adapters(q2, k2, v2))
    group.launch_down()
    got = ops_mod.rope_attn_decode(q2, k2, v2, kc2, vc2, t["cos"], t["sin"], mask, pos, c["scaling"], lora=group)
    torch.cuda.synchronize()
    assert torch.equal(q2, t["q"]) and torch.equal(k2, t["k"]) and torch.equal(v2, t["v"])   # inputs untouched
    assert not torch.equal(q1, t["q"]) or "q" not in which
    for a, b in ((kc2, kc1), (vc2, vc1)):
        assert torch.equal(a[:, :, :p], b[:, :, :p]) and torch.equal(a[:, :, p + 1:], b[:, :, p + 1:])
        within_one_step_of(bf16_to_bits(a[:, :, p]), bf16_to_bits(b[:, :, p]), bf16_to_bits(b[:, :, p]))
        assert (a[:, :, p] != b[:, :, p]).float().mean().item() < 0.02
    diff = (got.float() - want.float()).abs()
    assert diff.max().item() <= 2.0 ** -6 * max(1.0, want.float().abs().max().item())
    assert (got != want).float().mean().item() < 0.05
    with pytest.raises(ValueError):   # a group over other outputs
        ops_mod.rope_attn_decode(q1, k1, v1, kc1, vc1, t["cos"], t["sin"], mask, pos, c["scaling"], lora=group)


@pytest.mark.parametrize("M,H,Hkv,D,fp32,r,with_qkv", [(2, 16, 16, 128, True, 32, True), (32, 16, 16, 128, True, 32, False),
                                                        (3, 8, 2, 64, False, 16, False), (5, 4, 4, 64, True, 64, True),
                                                        (9, 16, 16, 128, False, 64, False), (4, 2, 1, 128, True, 8, False)])
def test_attention_leaves_the_output_adapters_down_projection(ops_mod, M, H, Hkv, D, fp32, r, with_qkv):
    """``rope_attn_decode(..., out_lora=group)``: the launch writes, per head, that head's share of
    ``out . A^T``; the heads' sum is the down-projection of the whole row (float64 over the bf16 output),
    the attention output itself is what the plain launch gives, and ``launch_up`` over the pieces equals the
    oracle's adapter applied to that output."""
    say("attention with output adapter", M, H, Hkv, D, fp32, r, with_qkv)
    L, p, N, K = 96, 57, 200, 256
    c = attn_case(500 + M, M, H, Hkv, D, L, p)
    dtype = torch.float32 if fp32 else torch.bfloat16
    t = {n: bits_to_bf16(c[n], DEV) for n in ("q", "k", "v", "cos", "sin")}
    mask = torch.from_numpy(c["mask"]).to(DEV)
    pos = torch.tensor([p], dtype=torch.int64, device=DEV)
    gen = torch.Generator().manual_seed(M + r)
    A = (torch.randn(r, H * D, generator=gen) * (H * D) ** -0.5).to(dtype).to(DEV)
    B = (torch.randn(N, r, generator=gen) * 0.2).to(dtype).to(DEV)
    y0 = rand_bits(np.random.default_rng(M), (M, N))
    y = bits_to_bf16(y0, DEV)
    out = torch.empty((M, H * D), dtype=torch.bfloat16, device=DEV)
    group = ops_mod.LoraAdd(out, [(A, B, 1.5, y)], parts=H)
    qkv = None
    if with_qkv:
        x = bits_to_bf16(rand_bits(np.random.default_rng(M + 1), (M, K)), DEV)
        Aq = (torch.randn(16, K, generator=gen) * K ** -0.5).to(dtype).to(DEV)
        Bq = (torch.randn(H * D, 16, generator=gen) * 0.2).to(dtype).to(DEV)
        qkv = ops_mod.LoraAdd(x, [(Aq, Bq, 2.0, t["q"])])
        qkv.launch_down()
    kc, vc = bits_to_bf16(c["kc"], DEV), bits_to_bf16(c["vc"], DEV)
    got = ops_mod.rope_attn_decode(t["q"], t["k"], t["v"], kc, vc, t["cos"], t["sin"], mask, pos, c["scaling"],
                                   out=out, lora=qkv, out_lora=group)
    kc2, vc2 = bits_to_bf16(c["kc"], DEV), bits_to_bf16(c["vc"], DEV)
    plain = ops_mod.rope_attn_decode(t["q"], t["k"], t["v"], kc2, vc2, t["cos"], t["sin"], mask, pos, c["scaling"],
                                     lora=qkv)
    torch.cuda.synchronize()
    # another build of the same kernel body: the compiler may fuse a multiply-add differently
    assert got.data_ptr() == out.data_ptr()
    print("  outputs that differ from the plain launch:", (got != plain).float().mean().item(),
          (got.float() - plain.float()).abs().max().item(), flush=True)
    within_one_step_of(bf16_to_bits(got), bf16_to_bits(plain), bf16_to_bits(plain))
    assert (got != plain).float().mean().item() < 0.01
    # the pieces: [M, H, r], head h from columns h*D .. (h+1)*D of the output
    o64 = out.float().cpu().numpy().astype(np.float64)
    A64 = A.float().cpu().numpy().astype(np.float64)
    pieces = group.t.cpu().numpy().astype(np.float64)
    assert pieces.shape == (M, H, r)
    want_pieces = np.einsum("mhd,jhd->mhj", o64.reshape(M, H, D), A64.reshape(r, H, D))
    scale = np.abs(o64).max() * np.abs(A64).max() * D
    assert np.abs(pieces - want_pieces).max() <= 2.0 ** -20 * scale
    assert np.abs(pieces.sum(axis=1) - o64 @ A64.T).max() <= 2.0 ** -18 * scale * H
    group.launch_up()
    torch.cuda.synchronize()
    want = d.lora_add(y0, bf16_to_bits(out), A.float().cpu().numpy(), B.float().cpu().numpy(), 1.5, fp32)
    within_one_step_of(bf16_to_bits(y), want, y0)
    with pytest.raises(ValueError):   # a group over another tensor than `out`
        ops_mod.rope_attn_decode(t["q"], t["k"], t["v"], kc2, vc2, t["cos"], t["sin"], mask, pos, c["scaling"],
                                 out_lora=group)


@pytest.mark.parametrize("M,K,Ns,ranks,fp32", [(2, 2048, (2048, 2048, 2048), (32, 32, 32), True),
                                               (32, 2048, (2048, 2048, 2048), (32, 32, 32), True),
                                               (7, 512, (96, 32), (8, 24), False), (16, 4096, (4096, 1024, 1024), (64, 16, 16), True),
                                               (20, 5632, (2048,), (16,), False), (1, 256, (48,), (8,), True)])
def test_down_projection_rides_with_the_base_launch(ops_mod, M, K, Ns, ranks, fp32):
    """``DirectGemv.launch(lora_down=group)``: the base projections equal the plain launch's and ``t`` the
    down-projection launch's, bit for bit (the same code, as extra workgroups of one launch; where the plain
    launch takes another split of K, to a rounding)."""
    from tests._util import to_device
    say("base launch with down-projection", M, K, Ns, ranks, fp32)
    rng = np.random.default_rng(M + K)
    dtype = torch.float32 if fp32 else torch.bfloat16
    x = bits_to_bf16(rand_bits(rng, (M, K)), DEV)
    gen = torch.Generator().manual_seed(K + M)
    packed, ads = [], []
    for i, (N, r) in enumerate(zip(Ns, ranks)):
        w = to_device(o.make_operands(900 + i, M, K, N, 128), DEV)
        packed.append(ops_mod.int4_prepack(w["qweight"], w["scales"], w["qzeros"], 128))
        A = (torch.randn(r, K, generator=gen) * K ** -0.5).to(dtype).to(DEV)
        B = (torch.randn(N, r, generator=gen) * 0.2).to(dtype).to(DEV)
        ads.append((A, B))
    plain = ops_mod.DirectGemv([(x, pw, False) for pw in packed])
    want_y = [y.clone() for y in plain.launch()]
    alone = ops_mod.LoraAdd(x, [(A, B, 1.0, y) for (A, B), y in zip(ads, want_y)])
    alone.launch_down()
    both = ops_mod.DirectGemv([(x, pw, False) for pw in packed])
    group = ops_mod.LoraAdd(x, [(A, B, 1.0, y) for (A, B), y in zip(ads, both.outputs)])
    group.t.fill_(float("nan"))
    got_y = both.launch(lora_down=group)
    torch.cuda.synchronize()
    for a, b in zip(got_y, want_y):
        if M > 16 and K > 4096:   # the plain launch of such rows splits K differently (register-fed, four waves)
            close = (a.float() - b.float()).abs() <= 2.0 ** -6 * b.float().abs() + 2.0 ** -7
            assert close.all() and (a != b).float().mean().item() < 0.02
        else:
            assert torch.equal(a, b)
    assert torch.equal(group.t, alone.t)
    t64 = x.float().cpu().numpy().astype(np.float64) @ np.concatenate(
        [A.float().cpu().numpy().astype(np.float64) for A, _ in ads]).T
    assert np.abs(group.t.cpu().numpy() - t64).max() <= (2.0 ** -7 if not fp32 else 2.0 ** -16) * max(1.0, np.abs(t64).max())


@pytest.mark.parametrize("M,K,Ns,ranks,fp32,with_residual", [
    (2, 2048, (2048, 2048, 2048), (32, 32, 32), True, False), (8, 2048, (2048, 512, 512), (32, 16, 16), True, True),
    (16, 2048, (2048, 2048, 2048), (32, 32, 32), False, True), (5, 640, (96, 48), (8, 24), False, False),
    (1, 1536, (64,), (64,), True, True)])
def test_norm_and_down_projection_ride_with_the_base_launch(ops_mod, M, K, Ns, ranks, fp32, with_residual):
    """``DirectGemv(norm=...).launch(lora_down=group)``: residual add, RMSNorm, the base projections and the
    adapters' down-projections of the normalised rows in one launch, against the norm launch followed by the
    base launch with its down-projection workgroups: the same ``h``, base outputs and ``t`` within what a last-bit
    difference in a row's scale (sums of squares added in another order) can move them."""
    from tests._util import to_device
    say("norm + base launch with down-projection", M, K, Ns, ranks, fp32, with_residual)
    rng = np.random.default_rng(3 * M + K)
    dtype = torch.float32 if fp32 else torch.bfloat16
    x, res = bits_to_bf16(rand_bits(rng, (M, K)), DEV), bits_to_bf16(rand_bits(rng, (M, K), 4.0), DEV)
    wn = bits_to_bf16(rand_bits(rng, (K,), 0.5), DEV)
    gen = torch.Generator().manual_seed(K + M)
    packed, ads = [], []
    for i, (N, r) in enumerate(zip(Ns, ranks)):
        w = to_device(o.make_operands(950 + i, M, K, N, 128), DEV)
        packed.append(ops_mod.int4_prepack(w["qweight"], w["scales"], w["qzeros"], 128))
        A = (torch.randn(r, K, generator=gen) * K ** -0.5).to(dtype).to(DEV)
        B = (torch.randn(N, r, generator=gen) * 0.2).to(dtype).to(DEV)
        ads.append((A, B))
    h_want, normed = ops_mod.add_rmsnorm(x, wn, 1e-6, res if with_residual else None)
    two = ops_mod.DirectGemv([(normed, pw, False) for pw in packed])
    g2 = ops_mod.LoraAdd(normed, [(A, B, 1.0, y) for (A, B), y in zip(ads, two.outputs)])
    want_y = [y.clone() for y in two.launch(lora_down=g2)]
    h_out = torch.zeros_like(x)
    one = ops_mod.DirectGemv([(x, pw, False) for pw in packed],
                             norm=(res if with_residual else None, wn, 1e-6, h_out if with_residual else None))
    g1 = ops_mod.LoraAdd(x, [(A, B, 1.0, y) for (A, B), y in zip(ads, one.outputs)])
    g1.t.fill_(float("nan"))
    got_y = one.launch(lora_down=g1)
    torch.cuda.synchronize()
    if with_residual:
        assert torch.equal(h_out, h_want)
    for a, b in zip(got_y, want_y):
        close = (a.float() - b.float()).abs() <= 2.0 ** -6 * b.float().abs() + 2.0 ** -7
        assert close.all() and (a != b).float().mean().item() < 0.02
    scale = max(1.0, g2.t.abs().max().item())
    assert torch.isfinite(g1.t).all() and (g1.t - g2.t).abs().max().item() <= 2.0 ** -6 * scale
    if M <= 16:
        with pytest.raises(ValueError):   # more rows than the adapters' workgroups keep in registers
            big = torch.zeros((17, K), dtype=torch.bfloat16, device=DEV)
            launch = ops_mod.DirectGemv([(big, packed[0], False)], norm=(None, wn, 1e-6, None))
            launch.launch(lora_down=ops_mod.LoraAdd(big, [(*ads[0], 1.0, launch.outputs[0])]))


@pytest.mark.parametrize("M,K,N,r,parts,fp32", [(2, 2048, 2048, 32, 16, True), (32, 2048, 2048, 32, 16, True),
                                                (7, 512, 100, 8, 1, False), (16, 4096, 4096, 64, 32, True),
                                                (20, 5632, 2048, 16, 3, False), (1, 256, 48, 8, 1, True),
                                                (32, 2048, 16384, 24, 2, True), (9, 11008, 64, 40, 1, False)])
def test_up_projection_joins_the_base_launch(ops_mod, M, K, N, r, parts, fp32):
    """``DirectGemv.launch(lora_up=group)`` against the two launches (base, then ``launch_up``) and
    against the oracle's adapter applied to the base launch's output."""
    from tests._util import to_device
    say("base launch with up-projection", M, K, N, r, parts, fp32)
    dtype = torch.float32 if fp32 else torch.bfloat16
    w = to_device(o.make_operands(700 + M, M, K, N, 128), DEV)
    x = w["x"]
    packed = ops_mod.int4_prepack(w["qweight"], w["scales"], w["qzeros"], 128)
    gen = torch.Generator().manual_seed(M + N)
    A = (torch.randn(r, K, generator=gen) * K ** -0.5).to(dtype).to(DEV)
    B = (torch.randn(N, r, generator=gen) * 0.2).to(dtype).to(DEV)
    pieces = (torch.randn(M, parts, r, generator=gen) * 0.5).to(DEV)   # any split of t: only the sum matters
    two = ops_mod.DirectGemv([(x, packed, False)])
    base = two.launch()[0].clone()
    g2 = ops_mod.LoraAdd(x, [(A, B, 1.5, two.outputs[0])], parts=parts)
    g2.t.copy_(pieces if parts > 1 else pieces[:, 0])
    g2.launch_up()
    one = ops_mod.DirectGemv([(x, packed, False)])
    g1 = ops_mod.LoraAdd(x, [(A, B, 1.5, one.outputs[0])], parts=parts)
    g1.t.copy_(g2.t)
    got = one.launch(lora_up=g1)[0]
    torch.cuda.synchronize()
    want = two.outputs[0]
    print("  outputs that differ from the two launches:", (got != want).float().mean().item(), flush=True)
    within_one_step_of(bf16_to_bits(got), bf16_to_bits(want), bf16_to_bits(base))
    assert (got != want).float().mean().item() < 0.01
    # against float64: base + 1.5 * (sum of the pieces, rounded for a bf16 adapter) . B^T
    t64 = pieces.double().sum(dim=1).cpu().numpy()
    if not fp32:
        t64 = o.bf16_bits_to_f32(o.f32_to_bf16_bits(pieces.sum(dim=1).cpu().numpy())).astype(np.float64)
    u = t64 @ B.double().cpu().numpy().T
    delta = u * 1.5 if fp32 else o.bf16_bits_to_f32(o.f32_to_bf16_bits(
        (o.bf16_bits_to_f32(o.f32_to_bf16_bits(u.astype(np.float32))) * np.float32(1.5)))).astype(np.float64)
    exact = o.f32_to_bf16_bits((base.float().cpu().numpy().astype(np.float64) + delta).astype(np.float32))
    within_one_step_of(bf16_to_bits(got), exact, bf16_to_bits(base))
    with pytest.raises(ValueError):
        one.launch(lora_up=g2)   # a group over another output


# ------------------------------------------------------------------ seeded random shapes through every decode-layer launch
@pytest.mark.parametrize("seed", [1, 2, 3])
def test_random_shapes(ops_mod, seed):
    """Twenty random cases per seed for each launch: ragged row counts, grouped-query heads, padding
    masks, positions anywhere in the cache, ranks and widths that do not divide the workgroup shapes."""
    from tests._util import assert_gemv_close, to_device

    rng = np.random.default_rng(seed)
    for case in range(20):
        M = int(rng.integers(1, 33))
        # residual add + norm, alone and inside an int4 launch
        K = int(rng.choice([128, 256, 640, 1024, 2048, 3072, 4096]))
        say("random", seed, case, "norm", M, K)
        x, res, wn = rand_bits(rng, (M, K)), rand_bits(rng, (M, K), 3.0), rand_bits(rng, (K,), 0.7)
        use_res = bool(rng.integers(0, 2))
        h_want, xn = d.add_rmsnorm(x, res if use_res else None, wn, 1e-5)
        xt, rt, wt = bits_to_bf16(x, DEV), bits_to_bf16(res, DEV), bits_to_bf16(wn, DEV)
        h, y = ops_mod.add_rmsnorm(xt, wt, 1e-5, rt if use_res else None)
        torch.cuda.synchronize()
        assert (bf16_to_bits(h) == h_want).all()
        assert ulp_distance(bf16_to_bits(y), xn).max() <= 1
        N = int(rng.integers(1, 20)) * 16 + int(rng.choice([0, 0, 4]))
        ops = o.make_operands(int(rng.integers(1 << 30)), M, K, N, 128)
        ops["x_bits"] = xn
        dd = to_device(ops, DEV)
        pw = ops_mod.int4_prepack(dd["qweight"], dd["scales"], dd["qzeros"], 128)
        h_out = torch.empty_like(xt)
        (yn,) = ops_mod.DirectGemv([(xt, pw, False)], norm=(rt if use_res else None, wt, 1e-5, h_out)).launch()
        torch.cuda.synchronize()
        assert (bf16_to_bits(h_out) == h_want).all()
        assert_gemv_close(bf16_to_bits(yn), ops, 128, f"random norm-fused {seed}/{case}")
        # attention
        D = int(rng.choice([64, 128]))
        Hkv = int(rng.choice([1, 2, 4]))
        H = Hkv * int(rng.choice([1, 2, 4]))
        L = int(rng.integers(1, 40)) * 8
        p = int(rng.integers(0, L))
        Ma = min(M, 8)
        say("random", seed, case, "attention", Ma, H, Hkv, D, L, p)
        c = attn_case(int(rng.integers(1 << 30)), Ma, H, Hkv, D, L, p)
        c["mask"] = (rng.random((Ma, L)) > 0.2).astype(np.uint8)
        c["mask"][:, p] = 1
        want, kc_want, vc_want = d.rope_attn_decode(c["q"], c["k"], c["v"], c["kc"], c["vc"], c["cos"], c["sin"],
                                                    c["mask"], p, H, Hkv, c["scaling"])
        out, kc, vc = run_attn(ops_mod, c)
        assert (bf16_to_bits(kc) == kc_want).all() and (bf16_to_bits(vc) == vc_want).all()
        got = o.bf16_bits_to_f32(bf16_to_bits(out)).astype(np.float64)
        tol = 0.51 * o.bf16_ulp(want.astype(np.float32)) + 2e-5 * np.abs(want).max()
        assert (np.abs(got - want) <= tol).all(), (seed, case, np.abs(got - want).max())
        # adapters
        r = int(rng.integers(1, 9)) * 8
        Nl = int(rng.integers(1, 300))
        fp32 = bool(rng.integers(0, 2))
        say("random", seed, case, "lora", M, K, Nl, r, fp32)
        dtype = torch.float32 if fp32 else torch.bfloat16
        A = torch.from_numpy((rng.standard_normal((r, K)) * K ** -0.5).astype(np.float32)).to(dtype)
        B = torch.from_numpy((rng.standard_normal((Nl, r)) * 0.1).astype(np.float32)).to(dtype)
        y0 = rand_bits(rng, (M, Nl), 2.0)
        yt = bits_to_bf16(y0, DEV)
        ops_mod.LoraAdd(xt, [(A.to(DEV), B.to(DEV), 1.5, yt)]).launch()
        torch.cuda.synchronize()
        within_one_step_of(bf16_to_bits(yt), d.lora_add(y0, x, A.float().numpy(), B.float().numpy(), 1.5, fp32), y0)
