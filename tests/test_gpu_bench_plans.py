"""The grouped launches the benchmark times, at their real size, against the oracle (MI355X).

``bench.build_set`` makes the operands exactly as ``bench.py`` does (seeded on the device, one
activation tensor per distinct input of a decoder layer), ``ops.GroupedGemv`` builds the plan the
benchmark launches (168 records at M = 1; 169 with the head at M = 32, walked in staged passes; 211
for the 7B-class shapes at M = 1, 8, 16), and every output of every record is compared with
``oracle.gemv_and_abs_f64`` under the operator tolerance, one matrix at a time.  Per plan the number of
outputs that pass only on the rule's extra term for cancelled sums is printed and capped
(``tests._util.MAX_FRACTION_BEYOND_STRICT``); no output at or above 2^-6 sum|x w| may need it at all.
"""

import sys

import numpy as np
import pytest
import torch

from oracle import int4_oracle as o
from tests._util import bf16_to_bits, check_gemv, report_tolerance

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
G = 128


def say(*a):
    print(*a, file=sys.stderr, flush=True)


def weights_to_host(it):
    return (it["qweight"].cpu().numpy(), bf16_to_bits(it["scales"]), it["qzeros"].cpu().numpy())


def run_and_check(items_by_rows, label):
    """``items_by_rows``: {M: items} over one set of weights (the same list order for every M)."""
    from visionrl_amd import ops

    plans = {}
    for M, items in items_by_rows.items():
        plans[M] = ops.GroupedGemv([(it["x"], it["prepacked"], False) for it in items])
        say(label, "rows", M, "records", plans[M].info.n_problems, "grid", plans[M].info.grid,
            "threads", plans[M].info.block_threads, "lds", plans[M].info.lds_bytes, "variant", plans[M].info.variant)
        first = [y.clone() for y in plans[M].launch()]
        plans[M].launch()
        torch.cuda.synchronize()
        assert all(torch.equal(a, b) for a, b in zip(first, plans[M].outputs)), "a second launch differs"
    rows = sorted(items_by_rows)
    n = len(items_by_rows[rows[0]])
    for i in range(n):
        qw, sc, qz = weights_to_host(items_by_rows[rows[0]][i])
        w = o.bf16_bits_to_f32(o.dequant_bf16(qw, sc, qz, G)).astype(np.float64)
        for M in rows:
            it = items_by_rows[M][i]
            x = o.bf16_bits_to_f32(bf16_to_bits(it["x"])).astype(np.float64)
            y = o.bf16_bits_to_f32(bf16_to_bits(plans[M].outputs[i])).astype(np.float64)
            check_gemv(y, x @ w.T, np.abs(x) @ np.abs(w).T, f"{label} M={M}: {it['name']}")
    for M in rows:
        report_tolerance(f"{label} M={M}", cap=True)


def test_janus_1b_step_m1():
    """Configuration 2: the 168-record plan of the headline figure."""
    import bench

    say("bench plan: Janus-Pro-1B set, M=1")
    items = bench.build_set(2, 1, torch.device(DEV), with_head=False)
    assert len(items) == 168
    run_and_check({1: items}, "config 2")


def test_janus_1b_step_m32_with_head():
    """Configuration 3: 169 records, 32 rows each, K = 5632 walked in staged passes."""
    import bench

    say("bench plan: Janus-Pro-1B set + head, M=32")
    items = bench.build_set(3, 32, torch.device(DEV), with_head=True)
    assert len(items) == 169
    run_and_check({32: items}, "config 3")


def test_7b_class_steps():
    """Configuration 4: 211 records at M = 1, 8 and 16 over one set of weights."""
    import bench

    say("bench plans: 7B-class set + head, M in (1, 8, 16)")
    dev = torch.device(DEV)
    base = bench.build_set(4, 16, dev, with_head=True, hidden=4096, inter=11008, layers=30, head=16384)
    assert len(base) == 211
    by_rows = {16: base}
    for M in (1, 8):   # the same weights under fewer activation rows; q|k|v and gate|up keep sharing a tensor
        cut = {}
        by_rows[M] = [dict(it, x=cut.setdefault(id(it["x"]), it["x"][:M].clone())) for it in base]
    run_and_check(by_rows, "config 4")
