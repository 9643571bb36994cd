"""The benchmark configurations at their full shapes, against the oracle (MI355X).

One matrix per distinct shape (the 24 / 30 layers of a configuration differ only in seed), through
the single-launch C-ABI entry points and through a grouped launch over prepacked weights.
"""

import sys

import numpy as np
import pytest
import torch

from oracle import int4_oracle as o
from tests._util import assert_gemv_close, bf16_to_bits, to_device

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def say(*a):
    print(*a, file=sys.stderr, flush=True)


@pytest.fixture(scope="module")
def ops_mod():
    from visionrl_amd import ops
    return ops


def check_both_paths(ops_mod, seed, M, K, N, G, mode="normal"):
    ops = o.make_operands(seed, M, K, N, G, mode)
    d = to_device(ops, DEV)
    y = ops_mod.int4_gemv(d["x"], d["qweight"], d["scales"], d["qzeros"], G)
    assert_gemv_close(bf16_to_bits(y), ops, G, f"single M{M} K{K} N{N} G{G}")
    if ops_mod.PrepackedWeight.supported(N, K, G):
        pw = ops_mod.int4_prepack(d["qweight"], d["scales"], d["qzeros"], G)
        grouped = ops_mod.GroupedGemv([(d["x"], pw, False)])
        (yp,) = grouped.launch()
        torch.cuda.synchronize()
        assert_gemv_close(bf16_to_bits(yp), ops, G, f"prepacked M{M} K{K} N{N} G{G}")
    return ops, d


# configuration 2 / 3: Janus-Pro-1B decoder shapes at M = 1 and M = 32, plus the image-token head
@pytest.mark.parametrize("M", [1, 32])
@pytest.mark.parametrize("K,N", [(2048, 2048), (2048, 5632), (5632, 2048), (2048, 16384)])
def test_janus_1b_shapes(ops_mod, M, K, N):
    say("janus-1b", M, K, N)
    check_both_paths(ops_mod, 2000 + M + K + N, M, K, N, 128)


# configuration 4: 7B-class shapes, M in {1, 8, 16}, head 4096 -> 16384
@pytest.mark.parametrize("M,K,N", [(1, 4096, 4096), (8, 4096, 11008), (16, 11008, 4096),
                                   (1, 11008, 4096), (16, 4096, 16384)])
def test_7b_class_shapes(ops_mod, M, K, N):
    say("7b-class", M, K, N)
    check_both_paths(ops_mod, 4000 + M + K + N, M, K, N, 128)


# configuration 5a: fused gate||up with the SiLU epilogue, K = 4096, N = 2 x 11008, M = 8
def test_fused_gate_up_7b(ops_mod):
    say("fused gate/up 7b")
    M, K, I, G = 8, 4096, 11008, 128
    ops = o.make_operands(5001, M, K, 2 * I, G)
    d = to_device(ops, DEV)
    args = (ops["x_bits"], ops["qweight"], ops["scales_bits"], ops["qzeros"], G)
    ref = o.gate_up_silu_f64(*args)
    acc, aabs = o.gemv_f64(*args), o.gemv_abs_f64(*args)
    g, u = acc[:, :I], acc[:, I:]
    sig = 1.0 / (1.0 + np.exp(-g))
    noise = 2.0 ** -18 * (np.abs(sig * (1.0 + g * (1.0 - sig)) * u) * aabs[:, :I]
                          + np.abs(o.silu_f64(g)) * aabs[:, I:])
    tol = np.maximum(o.bf16_ulp(ref), 1e-2 * np.abs(ref)) + noise
    y = ops_mod.int4_gate_up_silu(d["x"], d["qweight"], d["scales"], d["qzeros"], G)
    err = np.abs(o.bf16_bits_to_f32(bf16_to_bits(y)).astype(np.float64) - ref)
    assert y.shape == (M, I) and (err <= tol).all()
    pw = ops_mod.int4_prepack(d["qweight"], d["scales"], d["qzeros"], G)
    (yp,) = ops_mod.GroupedGemv([(d["x"], pw, True)]).launch()
    torch.cuda.synchronize()
    err = np.abs(o.bf16_bits_to_f32(bf16_to_bits(yp)).astype(np.float64) - ref)
    assert (err <= tol).all()


# configuration 5b: group-size sweep with log-uniform scales and asymmetric zero-points
@pytest.mark.parametrize("G", [32, 64, 128])
def test_group_size_sweep(ops_mod, G):
    say("group sweep", G)
    ops, d = check_both_paths(ops_mod, 5100 + G, 1, 5632, 2048, G, "loguniform")
    w = bf16_to_bits(ops_mod.int4_dequant(d["qweight"], d["scales"], d["qzeros"], G))
    assert (w == o.dequant_bf16(ops["qweight"], ops["scales_bits"], ops["qzeros"], G)).all()


def test_whole_decode_step_in_one_launch(ops_mod):
    """Two layers' worth of the configuration-2 set in one grouped launch: every output of every
    problem against the oracle, and a second launch reproduces the first bit for bit."""
    say("grouped decode set")
    shapes = [(2048, 2048)] * 4 + [(2048, 5632)] * 2 + [(5632, 2048)]
    problems, checks = [], []
    xs = {}
    for layer in range(2):
        for j, (K, N) in enumerate(shapes):
            ops = o.make_operands(2000 + 10 * layer + j, 1, K, N, 128)
            if K in xs:                       # one activation vector per K, as in the benchmark
                ops["x_bits"] = xs[K][0]
            d = to_device(ops, DEV)
            if K in xs:
                d["x"] = xs[K][1]
            else:
                xs[K] = (ops["x_bits"], d["x"])
            problems.append((d["x"], ops_mod.int4_prepack(d["qweight"], d["scales"], d["qzeros"], 128), False))
            checks.append(ops)
    grouped = ops_mod.GroupedGemv(problems)
    outs = grouped.launch()
    torch.cuda.synchronize()
    for y, ops in zip(outs, checks):
        assert_gemv_close(bf16_to_bits(y), ops, 128, "decode set")
    first = [y.clone() for y in outs]
    grouped.launch()
    torch.cuda.synchronize()
    assert all(torch.equal(a, b) for a, b in zip(first, grouped.outputs))


def test_vector_unit_dot_build_of_the_grouped_launch(ops_mod):
    """The comparison build (dot product by v_dot2_f32_bf16 instead of the matrix cores): the same
    dequantised weights bit for bit (one-hot activations return a column of the tile) and outputs
    within the operator tolerance, over a plan with more tiles than the device has workgroup slots."""
    say("grouped launch, vector-unit dot product")
    shapes = [(2048, 2048)] * 4 + [(2048, 5632)] * 2 + [(5632, 2048)]
    problems, checks = [], []
    for layer in range(6):
        for j, (K, N) in enumerate(shapes):
            ops = o.make_operands(2300 + 10 * layer + j, 1, K, N, 128)
            if layer == 0:                       # x = e_k: the output row is column k of the dequantised tile
                k = (37 * j + 5) % K
                ops["x_bits"] = np.zeros((1, K), dtype=np.uint16)
                ops["x_bits"][0, k] = 0x3F80
            d = to_device(ops, DEV)
            problems.append((d["x"], ops_mod.int4_prepack(d["qweight"], d["scales"], d["qzeros"], 128), False))
            checks.append((ops, (37 * j + 5) % K if layer == 0 else None))
    from bench import ValuDotLaunch   # the build lives in the measurement library

    grouped = ValuDotLaunch(problems)
    outs = grouped.launch()
    torch.cuda.synchronize()
    for y, (ops, k) in zip(outs, checks):
        assert_gemv_close(bf16_to_bits(y), ops, 128, "vector-unit dot")
        if k is not None:
            w = o.dequant_bf16(ops["qweight"], ops["scales_bits"], ops["qzeros"], 128)
            assert (bf16_to_bits(y)[0] == w[:, k]).all()
    with pytest.raises(ValueError):             # one activation row only
        x2 = torch.zeros((2, 2048), dtype=torch.bfloat16, device=DEV)
        ValuDotLaunch([(x2, problems[0][1], False)] * 600)
