"""Seeded random shapes through every launch path against the oracle.

Small operands, many combinations: ragged N, K that is a multiple of 128 but not of 512, group sizes
32/64/128, 1..40 activation rows, fused and plain, alone and as the middle record of a three-record plan.
"""
import random

import numpy as np
import pytest
import torch

from oracle import int4_oracle as o
from tests._util import bf16_to_bits, to_device

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def within_tolerance(y, d, G, fused):
    args = (d["x_bits"], d["qweight"], d["scales_bits"], d["qzeros"], G)
    got = o.bf16_bits_to_f32(bf16_to_bits(y)).astype(np.float64)
    if fused:
        ref = o.gate_up_silu_f64(*args)
        tol = np.maximum(2 * o.bf16_ulp(ref), 1e-2 * np.abs(ref)) + 1e-5
    else:
        ref = o.gemv_f64(*args)
        tol = o.gemv_tolerance(ref, o.gemv_abs_f64(*args))
    return got.shape == ref.shape and bool((np.abs(got - ref) <= tol).all())


@pytest.mark.parametrize("seed", [0, 1, 2])
def test_random_shapes_all_paths(seed):
    from visionrl_amd import ops

    rnd = random.Random(seed)
    failures = []
    for case in range(40):
        G = rnd.choice([32, 64, 128, 128, 128])
        K = 128 * rnd.randint(1, 24)
        fused = rnd.random() < 0.25
        N = 32 * rnd.randint(1, 12) if fused else rnd.randint(1, 200)
        M = rnd.choice([1, 1, 2, 3, 7, 8, 15, 16, 17, 31, 32, 40])
        mode = rnd.choice(["normal", "loguniform"])
        tag = f"seed {seed} case {case}: M={M} K={K} N={N} G={G} fused={fused} {mode}"
        print("[case]", tag, flush=True)
        d = o.make_operands(50000 + 100 * seed + case, M, K, N, G, mode)
        t = to_device(d, DEV)
        pw = ops.int4_prepack(t["qweight"], t["scales"], t["qzeros"], G)
        d2 = o.make_operands(60000 + 100 * seed + case, min(M, 16), 128 * rnd.randint(1, 12), rnd.randint(1, 90), G)
        t2 = to_device(d2, DEV)
        pw2 = ops.int4_prepack(t2["qweight"], t2["scales"], t2["qzeros"], G)

        results = {"grouped": ops.GroupedGemv([(t["x"], pw, fused)]).launch()[0]}
        outs = ops.GroupedGemv([(t2["x"], pw2, False), (t["x"], pw, fused), (t2["x"], pw2, False)]).launch()
        results["grouped, middle of three"] = outs[1]
        if M <= pw.direct_rows(fused):
            results["plan-free"] = ops.DirectGemv([(t["x"], pw, fused)]).launch()[0]
        if fused:
            results["canonical single"] = ops.int4_gate_up_silu(t["x"], t["qweight"], t["scales"], t["qzeros"], G)
        else:
            results["canonical single"] = ops.int4_gemv(t["x"], t["qweight"], t["scales"], t["qzeros"], G)
        if M <= 16:
            results["canonical grouped"] = ops.GroupedGemv(
                [(t["x"], t["qweight"], t["scales"], t["qzeros"], G, fused)]).launch()[0]
        torch.cuda.synchronize()
        for name, y in results.items():
            if not within_tolerance(y, d, G, fused):
                failures.append(f"{tag}: {name}")
        for y in (outs[0], outs[2]):
            if not within_tolerance(y, d2, G, False):
                failures.append(f"{tag}: neighbour record of the plan")
    assert not failures, failures
