"""Parity of the HIP path against the CPU oracle, on an MI355X.

Every call goes through the torch operators, i.e. through the C ABI.  Dequant is
checked bit for bit; GEMV outputs against the float64 truth under the operator
tolerance (see ``tests/_util.assert_gemv_close``); the in-kernel dequant of the
GEMV is also checked bit for bit through one-hot activations.
"""

import sys

import numpy as np
import pytest
import torch

from oracle import int4_oracle as o
from tests._util import assert_gate_up_close, assert_gemv_close, bf16_to_bits, bits_to_bf16, to_device

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def say(*a):
    print(*a, file=sys.stderr, flush=True)


@pytest.fixture(scope="module")
def ops_mod():
    from visionrl_amd import ops
    return ops


def run_gemv(ops_mod, ops, G):
    d = to_device(ops, DEV)
    y = ops_mod.int4_gemv(d["x"], d["qweight"], d["scales"], d["qzeros"], G)
    torch.cuda.synchronize()
    return bf16_to_bits(y)


# ------------------------------------------------------------------ dequant
def test_dequant_exhaustive_bit_exact(ops_mod):
    """All 256 (q, z) pairs x every bf16 mantissa at several exponents."""
    say("dequant exhaustive")
    mant = np.arange(128, dtype=np.uint16)
    scales = np.concatenate([(e << 7) | mant for e in (0x01, 0x60, 0x70, 0x78, 0x7F, 0x90)])
    scales = np.concatenate([scales, scales | 0x8000]).astype(np.uint16)   # negative scales too
    G = 16
    rows = [(int(sb), z) for sb in scales for z in range(16)]
    N = len(rows)
    q = np.tile(np.arange(16, dtype=np.uint8), (N, 1))
    z = np.array([r[1] for r in rows], dtype=np.uint8)[:, None]
    sb = np.array([r[0] for r in rows], dtype=np.uint16)[:, None]
    qweight, qzeros = o.pack_nibbles(q), o.pack_nibbles(z)
    want = o.dequant_bf16(qweight, sb, qzeros, G)
    got = ops_mod.int4_dequant(torch.from_numpy(qweight).to(DEV), bits_to_bf16(sb, DEV),
                               torch.from_numpy(qzeros).to(DEV), G)
    got = bf16_to_bits(got)
    # +0 and -0 are the same weight
    same = (got == want) | (((got | want) & 0x7FFF) == 0)
    assert same.all(), f"{int((~same).sum())} mismatches"


@pytest.mark.parametrize("N,K,G,mode", [
    (64, 2048, 128, "normal"), (33, 5632, 32, "loguniform"), (17, 5632, 64, "loguniform"),
    (5, 88, 8, "normal"), (256, 4096, 128, "normal"), (7, 48, 24, "normal"),
])
def test_dequant_random_bit_exact(ops_mod, N, K, G, mode):
    say("dequant", N, K, G, mode)
    ops = o.make_operands(200 + N, 1, K, N, G, mode)
    d = to_device(ops, DEV)
    got = bf16_to_bits(ops_mod.int4_dequant(d["qweight"], d["scales"], d["qzeros"], G))
    want = o.dequant_bf16(ops["qweight"], ops["scales_bits"], ops["qzeros"], G)
    assert (got == want).all()


# ------------------------------------------------------------------ GEMV
TILE_SHAPES = [
    # M, K, N, G  (K % 128 == 0 and G % 32 == 0: the MFMA tile path)
    (1, 2048, 2048, 128),      # configuration 1
    (1, 128, 16, 128),
    (1, 256, 40, 32),          # ragged N
    (2, 384, 16, 64),
    (3, 1024, 100, 128),
    (7, 2048, 33, 64),
    (16, 2048, 256, 128),
    (16, 5632, 64, 128),       # staged activations take several passes
    (17, 1024, 48, 128),       # second slab of activation rows
    (32, 2048, 512, 128),      # rollout batch
    (1, 5632, 2048, 32),       # configuration 5b
    (1, 5632, 2048, 64),
    (1, 5632, 2048, 128),
    (8, 4096, 300, 128),
    (1, 2048, 5632, 128),
    (1, 11008, 96, 128),
]


@pytest.mark.parametrize("M,K,N,G", TILE_SHAPES)
def test_gemv_tile_path(ops_mod, M, K, N, G):
    say("gemv tile", M, K, N, G)
    mode = "loguniform" if K == 5632 and N == 2048 else "normal"
    ops = o.make_operands(1000 + 7 * M + K + N + G, M, K, N, G, mode)
    be = assert_gemv_close(run_gemv(ops_mod, ops, G), ops, G, f"M{M} K{K} N{N} G{G}")
    say("  worst |err| / sum|x w| (includes the output rounding)", be)


GENERIC_SHAPES = [
    (1, 8, 1, 8), (1, 64, 5, 8), (2, 88, 9, 8), (3, 48, 7, 24), (1, 192, 33, 16),
    (5, 96, 4, 32), (9, 200, 11, 40), (1, 2040, 16, 8),
]


@pytest.mark.parametrize("M,K,N,G", GENERIC_SHAPES)
def test_gemv_generic_path(ops_mod, M, K, N, G):
    say("gemv generic", M, K, N, G)
    ops = o.make_operands(2000 + M + K + N + G, M, K, N, G)
    assert_gemv_close(run_gemv(ops_mod, ops, G), ops, G, f"M{M} K{K} N{N} G{G}")


@pytest.mark.parametrize("M,K,N,G", [(1, 256, 48, 128), (4, 512, 32, 32), (1, 96, 8, 8)])
def test_gemv_one_hot_is_the_exact_weight_column(ops_mod, M, K, N, G):
    """x = e_k in every activation row: y must equal column k of the canonical tile bit for bit,
    which pins the in-register dequant of the GEMV kernels (no summation error is possible)."""
    say("gemv one-hot", M, K, N, G)
    ops = o.make_operands(3000 + K, M, K, N, G, "loguniform")
    w = o.dequant_bf16(ops["qweight"], ops["scales_bits"], ops["qzeros"], G)
    ks = sorted(set([0, 1, 4, 7, 8, 31, 32, 33, K // 2 + 5, K - 9, K - 1]))
    for k0 in ks:
        x = np.zeros((M, K), dtype=np.float32)
        for m in range(M):
            x[m, (k0 + 13 * m) % K] = 1.0
        ops["x_bits"] = o.f32_to_bf16_bits(x)
        y = run_gemv(ops_mod, ops, G)
        for m in range(M):
            want = w[:, (k0 + 13 * m) % K]
            same = (y[m] == want) | (((y[m] | want) & 0x7FFF) == 0)
            assert same.all(), (k0, m)


def test_gemv_every_q_z_pair_through_the_kernel(ops_mod):
    """All 256 (q, z) pairs x 128 mantissas through the tile kernel's dequant, via one-hot x."""
    say("gemv exhaustive one-hot")
    G, K = 32, 128
    mant = np.arange(128, dtype=np.uint16)
    scales = np.concatenate([(e << 7) | mant for e in (0x70, 0x78)]).astype(np.uint16)
    rows = [(int(sb), z) for sb in scales for z in range(16)]
    N = len(rows)
    q = np.tile(np.arange(16, dtype=np.uint8), (N, K // 16))
    z = np.repeat(np.array([r[1] for r in rows], dtype=np.uint8)[:, None], K // G, axis=1)
    sb = np.repeat(np.array([r[0] for r in rows], dtype=np.uint16)[:, None], K // G, axis=1)
    ops = {"qweight": o.pack_nibbles(q), "scales_bits": sb, "qzeros": o.pack_nibbles(z)}
    w = o.dequant_bf16(ops["qweight"], sb, ops["qzeros"], G)
    x = np.zeros((16, K), dtype=np.float32)
    for m in range(16):
        x[m, 16 * (m % 8) + m] = 1.0      # activation row m selects k with q = m
    ops["x_bits"] = o.f32_to_bf16_bits(x)
    y = run_gemv(ops_mod, ops, G)
    for m in range(16):
        want = w[:, 16 * (m % 8) + m]
        same = (y[m] == want) | (((y[m] | want) & 0x7FFF) == 0)
        assert same.all(), m


def test_gemv_integer_case_is_exact(ops_mod):
    """s = 1, z = 0, x in {-1,0,1}: an integer matmul, exact in fp32, so only the output rounds."""
    say("gemv integer")
    M, K, N, G = 5, 1024, 80, 128
    rng = np.random.default_rng(5)
    q = rng.integers(0, 16, (N, K), dtype=np.uint8)
    x = rng.integers(-1, 2, (M, K)).astype(np.float32)
    ops = {"x_bits": o.f32_to_bf16_bits(x), "qweight": o.pack_nibbles(q),
           "scales_bits": o.f32_to_bf16_bits(np.ones((N, K // G), dtype=np.float32)),
           "qzeros": o.pack_nibbles(np.zeros((N, K // G), dtype=np.uint8))}
    want = (x.astype(np.int64) @ q.astype(np.int64).T).astype(np.float32)
    assert (run_gemv(ops_mod, ops, G) == o.f32_to_bf16_bits(want)).all()


def test_gemv_zero_when_q_equals_z(ops_mod):
    say("gemv q==z")
    M, K, N, G = 2, 512, 64, 64
    ops = o.make_operands(6, M, K, N, G)
    ops["qweight"] = o.pack_nibbles(np.repeat(ops["z"], G, axis=1))
    assert ((run_gemv(ops_mod, ops, G) & 0x7FFF) == 0).all()


def test_gemv_rows_are_independent_of_batch(ops_mod):
    """Row m of a batched call equals the single-row call (same kernel arithmetic per row)."""
    say("gemv batch consistency")
    M, K, N, G = 32, 2048, 128, 128
    ops = o.make_operands(7, M, K, N, G)
    full = run_gemv(ops_mod, ops, G)
    for m in (0, 5, 15, 16, 31):
        one = dict(ops)
        one["x_bits"] = ops["x_bits"][m:m + 1]
        single = run_gemv(ops_mod, one, G)
        tol_ops = dict(ops)
        tol_ops["x_bits"] = ops["x_bits"][m:m + 1]
        assert_gemv_close(single, tol_ops, G, f"row {m} alone")
        diff = np.abs(o.bf16_bits_to_f32(single[0]).astype(np.float64)
                      - o.bf16_bits_to_f32(full[m]).astype(np.float64))
        assert (diff <= o.bf16_ulp(o.bf16_bits_to_f32(full[m]).astype(np.float64))).all()


def test_gemv_linearity_in_x(ops_mod):
    say("gemv linearity")
    K, N, G = 2048, 256, 128
    ops = o.make_operands(8, 1, K, N, G)
    y1 = run_gemv(ops_mod, ops, G)
    two = dict(ops)
    two["x_bits"] = o.f32_to_bf16_bits(o.bf16_bits_to_f32(ops["x_bits"]) * 2.0)
    y2 = run_gemv(ops_mod, two, G)
    # doubling x doubles every partial sum exactly, so the bf16 results differ by one exponent step
    assert (o.bf16_bits_to_f32(y2) == 2.0 * o.bf16_bits_to_f32(y1)).all()


def test_gemv_is_deterministic(ops_mod):
    say("gemv determinism")
    ops = o.make_operands(9, 4, 2048, 2048, 128)
    a = run_gemv(ops_mod, ops, 128)
    b = run_gemv(ops_mod, ops, 128)
    assert (a == b).all()


# ------------------------------------------------------------------ fused gate/up
@pytest.mark.parametrize("M,K,I,G", [
    (1, 2048, 5632, 128), (8, 4096, 704, 128), (3, 256, 24, 64), (16, 1024, 50, 32),
    (2, 88, 6, 8), (20, 512, 40, 128),
])
def test_gate_up_silu(ops_mod, M, K, I, G):
    say("gate_up_silu", M, K, I, G)
    ops = o.make_operands(4000 + M + K + I, M, K, 2 * I, G)
    d = to_device(ops, DEV)
    y = bf16_to_bits(ops_mod.int4_gate_up_silu(d["x"], d["qweight"], d["scales"], d["qzeros"], G))
    args = (ops["x_bits"], ops["qweight"], ops["scales_bits"], ops["qzeros"], G)
    ref = o.gate_up_silu_f64(*args)
    acc = o.gemv_f64(*args)
    aabs = o.gemv_abs_f64(*args)
    # first-order propagation of the accumulation noise through silu(g) * u
    g, u = acc[:, :I], acc[:, I:]
    sig = 1.0 / (1.0 + np.exp(-g))
    dsilu = sig * (1.0 + g * (1.0 - sig))
    noise = 2.0 ** -18 * (np.abs(dsilu * u) * aabs[:, :I] + np.abs(o.silu_f64(g)) * aabs[:, I:])
    tol = np.maximum(o.bf16_ulp(ref), 1e-2 * np.abs(ref)) + noise
    err = np.abs(o.bf16_bits_to_f32(y).astype(np.float64) - ref)
    assert y.shape == (M, I)
    assert (err <= tol).all(), f"{int((err > tol).sum())} of {err.size} out of tolerance"


# ------------------------------------------------------------------ grouped launch
def test_grouped_launch_matches_single_launches(ops_mod):
    say("grouped")
    shapes = [(1, 2048, 2048, 128, False), (1, 2048, 2048, 128, False), (1, 2048, 5632, 128, False),
              (1, 5632, 2048, 128, False), (4, 2048, 200, 64, False), (2, 1024, 2 * 96, 128, True)]
    problems, singles, all_ops = [], [], []
    for i, (M, K, N, G, fused) in enumerate(shapes):
        ops = o.make_operands(5000 + i, M, K, N, G)
        d = to_device(ops, DEV)
        problems.append((d["x"], d["qweight"], d["scales"], d["qzeros"], G, fused))
        fn = ops_mod.int4_gate_up_silu if fused else ops_mod.int4_gemv
        singles.append(fn(d["x"], d["qweight"], d["scales"], d["qzeros"], G))
        all_ops.append((ops, G, fused))
    grouped = ops_mod.GroupedGemv(problems)
    for rep in range(2):
        for y in grouped.outputs:
            y.zero_()
        outs = grouped.launch()
        torch.cuda.synchronize()
        for y, ref, (ops, G, fused) in zip(outs, singles, all_ops):
            assert y.shape == ref.shape
            if not fused:
                assert_gemv_close(bf16_to_bits(y), ops, G, "grouped")
            diff = (y.float() - ref.float()).abs()
            ulp = torch.from_numpy(o.bf16_ulp(ref.float().cpu().numpy().astype(np.float64))).to(DEV)
            assert (diff <= ulp).all()


# ------------------------------------------------------------------ prepacked weights
PP_SHAPES = [
    # M, K, N, fused
    (1, 2048, 2048, False), (1, 5632, 2048, False), (1, 2048, 5632, False),
    (1, 128, 16, False),        # K padded from 128 to 512
    (3, 640, 50, False),        # ragged N and K
    (16, 2048, 256, False), (16, 5632, 64, False),   # the second needs staged passes
    (7, 11008, 96, False),      # 21.5 super-chunks
    (20, 1024, 48, False),      # 17..32 rows: two MFMA row blocks per weight tile
    (32, 2048, 512, False),     # rollout batch, x staged whole in a 16-wave workgroup
    (32, 5632, 96, False),      # rollout batch with staged passes over K
    (40, 512, 32, False),       # more than 32 rows: two records
    (12, 4096, 64, False),      # 8-wave workgroups
    (1, 2048, 2 * 5632, True), (8, 4096, 2 * 704, True), (16, 1024, 2 * 48, True),
    (32, 2048, 2 * 64, True),
]


def run_grouped(ops_mod, problems):
    grouped = ops_mod.GroupedGemv(problems)
    outs = grouped.launch()
    torch.cuda.synchronize()
    return grouped, outs


@pytest.mark.parametrize("M,K,N,fused", PP_SHAPES)
def test_prepacked_grouped_parity(ops_mod, M, K, N, fused):
    say("prepacked", M, K, N, fused)
    G = 128
    ops = o.make_operands(6000 + M + K + N, M, K, N, G)
    d = to_device(ops, DEV)
    pw = ops_mod.int4_prepack(d["qweight"], d["scales"], d["qzeros"], G)
    _, (y,) = run_grouped(ops_mod, [(d["x"], pw, fused)])
    if not fused:
        assert_gemv_close(bf16_to_bits(y), ops, G, f"prepacked M{M} K{K} N{N}")
        return
    args = (ops["x_bits"], ops["qweight"], ops["scales_bits"], ops["qzeros"], G)
    ref = o.gate_up_silu_f64(*args)
    ref_op = o.bf16_bits_to_f32(o.gate_up_silu_bf16(*args)).astype(np.float64)
    got = o.bf16_bits_to_f32(bf16_to_bits(y)).astype(np.float64)
    assert got.shape == ref.shape
    # against the float64 truth: bf16 tolerance plus two ulps for the fp32 epilogue of near-cancelling sums
    tol = np.maximum(2 * o.bf16_ulp(ref), 1e-2 * np.abs(ref)) + 1e-5
    assert (np.abs(got - ref) <= tol).all()
    assert (np.abs(got - ref_op) <= tol).all()


@pytest.mark.parametrize("M,K,N", [(32, 1024, 144), (1, 512, 80), (16, 2048, 112)])
def test_prepacked_records_sharing_activations(ops_mod, M, K, N):
    """Records side by side that read the same x (q|k|v, gate|up) keep it staged; a record
    with another x between them, or after them, stages its own.  Few tiles per record, so that
    every workgroup's range runs over several records."""
    say("shared x", M, K, N)
    G = 128
    sets = [o.make_operands(6500 + 10 * i + M, M, K, N, G) for i in range(6)]
    x1 = bits_to_bf16(sets[0]["x_bits"], DEV)
    x2 = bits_to_bf16(sets[2]["x_bits"], DEV)
    which = [0, 0, 2, 0, 0, 2]                       # whose activations record i multiplies
    problems = []
    for i, ops in enumerate(sets):
        d = to_device(ops, DEV)
        pw = ops_mod.int4_prepack(d["qweight"], d["scales"], d["qzeros"], G)
        problems.append(((x1, x2)[which[i] // 2], pw, False))
    _, ys = run_grouped(ops_mod, problems)
    for i, (ops, y) in enumerate(zip(sets, ys)):
        ref = dict(ops)
        ref["x_bits"] = sets[which[i]]["x_bits"]
        assert_gemv_close(bf16_to_bits(y), ref, G, f"record {i} of 6, M{M} K{K} N{N}")


@pytest.mark.parametrize("M,K,N", [(1, 512, 32), (4, 1024, 48), (16, 640, 16)])
def test_prepacked_one_hot_is_the_exact_weight_column(ops_mod, M, K, N):
    """The matrix-core dequant of the prepacked path reproduces the canonical tile bit for bit."""
    say("prepacked one-hot", M, K, N)
    G = 128
    ops = o.make_operands(7000 + K, M, K, N, G, "loguniform")
    w = o.dequant_bf16(ops["qweight"], ops["scales_bits"], ops["qzeros"], G)
    d = to_device(ops, DEV)
    pw = ops_mod.int4_prepack(d["qweight"], d["scales"], d["qzeros"], G)
    for k0 in sorted(set([0, 1, 3, 4, 7, 8, 31, 32, 127, 128, 129, K // 2 + 5, K - 9, K - 1])):
        x = np.zeros((M, K), dtype=np.float32)
        for m in range(M):
            x[m, (k0 + 29 * m) % K] = 1.0
        xd = bits_to_bf16(o.f32_to_bf16_bits(x), DEV)
        _, (y,) = run_grouped(ops_mod, [(xd, pw, False)])
        y = bf16_to_bits(y)
        for m in range(M):
            want = w[:, (k0 + 29 * m) % K]
            same = (y[m] == want) | (((y[m] | want) & 0x7FFF) == 0)
            assert same.all(), (k0, m)


def test_prepacked_every_q_z_pair(ops_mod):
    """All 256 (q, z) pairs x every bf16 mantissa at three exponents through the 4x4x4 dequant."""
    say("prepacked exhaustive one-hot")
    G, K = 128, 128
    mant = np.arange(128, dtype=np.uint16)
    scales = np.concatenate([(e << 7) | mant for e in (0x60, 0x78, 0x7C)]).astype(np.uint16)
    scales = np.concatenate([scales, scales[:128] | 0x8000])
    rows = [(int(sb), z) for sb in scales for z in range(16)]
    N = len(rows)
    q = np.tile(np.arange(16, dtype=np.uint8), (N, K // 16))
    z = np.array([r[1] for r in rows], dtype=np.uint8)[:, None]
    sb = np.array([r[0] for r in rows], dtype=np.uint16)[:, None]
    ops = {"qweight": o.pack_nibbles(q), "scales_bits": sb, "qzeros": o.pack_nibbles(z)}
    w = o.dequant_bf16(ops["qweight"], sb, ops["qzeros"], G)
    x = np.zeros((16, K), dtype=np.float32)
    for m in range(16):
        x[m, 16 * (m % 8) + m] = 1.0      # activation row m selects a k with q = m
    pw = ops_mod.int4_prepack(torch.from_numpy(ops["qweight"]).to(DEV), bits_to_bf16(sb, DEV),
                              torch.from_numpy(ops["qzeros"]).to(DEV), G)
    _, (y,) = run_grouped(ops_mod, [(bits_to_bf16(o.f32_to_bf16_bits(x), DEV), pw, False)])
    y = bf16_to_bits(y)
    for m in range(16):
        want = w[:, 16 * (m % 8) + m]
        same = (y[m] == want) | (((y[m] | want) & 0x7FFF) == 0)
        assert same.all(), m


def test_prepacked_and_canonical_records_in_one_plan(ops_mod):
    say("prepacked mixed plan")
    G = 128
    problems, checks = [], []
    for i, (M, K, N, pp) in enumerate([(1, 2048, 2048, True), (1, 2048, 2048, False), (2, 5632, 512, True),
                                       (1, 2048, 100, False)]):
        ops = o.make_operands(8000 + i, M, K, N, G)
        d = to_device(ops, DEV)
        if pp:
            problems.append((d["x"], ops_mod.int4_prepack(d["qweight"], d["scales"], d["qzeros"], G), False))
        else:
            problems.append((d["x"], d["qweight"], d["scales"], d["qzeros"], G, False))
        checks.append(ops)
    grouped, outs = run_grouped(ops_mod, problems)
    for y, ops in zip(outs, checks):
        assert_gemv_close(bf16_to_bits(y), ops, G, "mixed plan")
    first = [y.clone() for y in outs]
    grouped.launch()
    torch.cuda.synchronize()
    assert all(torch.equal(a, b) for a, b in zip(first, grouped.outputs))


def test_prepack_rejects_other_group_sizes(ops_mod):
    ops = o.make_operands(11, 1, 256, 16, 16)
    d = to_device(ops, DEV)
    assert not ops_mod.PrepackedWeight.supported(16, 256, 16)
    assert not ops_mod.PrepackedWeight.supported(16, 256, 256)
    with pytest.raises(ValueError):
        ops_mod.int4_prepack(d["qweight"], d["scales"], d["qzeros"], 16)


PP_GROUP_SHAPES = [
    # M, K, N, G, fused
    (1, 5632, 2048, 32, False), (1, 5632, 2048, 64, False),     # the group-size sweep configuration
    (1, 128, 16, 32, False), (3, 640, 50, 64, False), (16, 2048, 256, 32, False),
    (32, 2048, 128, 64, False), (32, 5632, 96, 32, False), (12, 4096, 64, 64, False),
    (1, 2048, 2 * 704, 64, True), (8, 1024, 2 * 48, 32, True),
]


@pytest.mark.parametrize("M,K,N,G,fused", PP_GROUP_SHAPES)
def test_prepacked_small_groups_parity(ops_mod, M, K, N, G, fused):
    """Group sizes 32 and 64 through the prepacked layout: grouped plan, and plan-free launch where it applies.
    Scales log-uniform over 1e-4..1e-1 with asymmetric zero-points, as in the sweep configuration."""
    say("prepacked groups", M, K, N, G, fused)
    ops = o.make_operands(9500 + M + K + N + G, M, K, N, G, "loguniform")
    d = to_device(ops, DEV)
    pw = ops_mod.int4_prepack(d["qweight"], d["scales"], d["qzeros"], G)
    results = [run_grouped(ops_mod, [(d["x"], pw, fused)])[1][0]]
    if M <= pw.direct_rows(fused):
        results.append(ops_mod.DirectGemv([(d["x"], pw, fused)]).launch()[0])
        torch.cuda.synchronize()
    args = (ops["x_bits"], ops["qweight"], ops["scales_bits"], ops["qzeros"], G)
    for y in results:
        if not fused:
            assert_gemv_close(bf16_to_bits(y), ops, G, f"prepacked G{G} M{M} K{K} N{N}")
            continue
        ref = o.gate_up_silu_f64(*args)
        got = o.bf16_bits_to_f32(bf16_to_bits(y)).astype(np.float64)
        tol = np.maximum(2 * o.bf16_ulp(ref), 1e-2 * np.abs(ref)) + 1e-5
        assert got.shape == ref.shape and (np.abs(got - ref) <= tol).all()


@pytest.mark.parametrize("G", [32, 64])
def test_prepacked_small_groups_one_hot_exact(ops_mod, G):
    """Every group boundary of the lane's 128-k span picks the right scale and zero-point, bit for bit."""
    say("prepacked groups one-hot", G)
    M, K, N = 4, 1024, 48
    ops = o.make_operands(9600 + G, M, K, N, G, "loguniform")
    w = o.dequant_bf16(ops["qweight"], ops["scales_bits"], ops["qzeros"], G)
    d = to_device(ops, DEV)
    pw = ops_mod.int4_prepack(d["qweight"], d["scales"], d["qzeros"], G)
    for k0 in sorted(set([0, 31, 32, 33, 63, 64, 65, 95, 96, 127, 128, 160, 511, 512, 544, K - 33, K - 1])):
        x = np.zeros((M, K), dtype=np.float32)
        for m in range(M):
            x[m, (k0 + 37 * m) % K] = 1.0
        xd = bits_to_bf16(o.f32_to_bf16_bits(x), DEV)
        outs = [run_grouped(ops_mod, [(xd, pw, False)])[1][0], ops_mod.DirectGemv([(xd, pw, False)]).launch()[0]]
        torch.cuda.synchronize()
        for y in outs:
            y = bf16_to_bits(y)
            for m in range(M):
                want = w[:, (k0 + 37 * m) % K]
                assert ((y[m] == want) | (((y[m] | want) & 0x7FFF) == 0)).all(), (G, k0, m)


def test_grouped_plan_takes_one_prepacked_group_size(ops_mod):
    """A throughput plan (more tiles than the latency kernel takes) holds prepacked records of one group size."""
    say("mixed group sizes")
    probs = []
    for i, G in enumerate((128, 64)):
        ops = o.make_operands(9700 + i, 1, 256, 16 * 2100, G)     # 2100 tiles each: beyond the latency mode
        d = to_device(ops, DEV)
        probs.append((d["x"], ops_mod.int4_prepack(d["qweight"], d["scales"], d["qzeros"], G), False))
    with pytest.raises(ValueError):
        ops_mod.GroupedGemv(probs)
    for p in probs:                                              # each alone is fine
        ops_mod.GroupedGemv([p]).launch()
    torch.cuda.synchronize()


# ------------------------------------------------------------------ contract violations
def test_operator_contract_errors(ops_mod):
    ops = o.make_operands(10, 2, 256, 16, 128)
    d = to_device(ops, DEV)
    with pytest.raises(TypeError):
        ops_mod.int4_gemv(d["x"].float(), d["qweight"], d["scales"], d["qzeros"], 128)
    with pytest.raises(ValueError):
        ops_mod.int4_gemv(d["x"][:, :128].contiguous(), d["qweight"], d["scales"], d["qzeros"], 128)
    with pytest.raises(ValueError):
        ops_mod.int4_gemv(d["x"].cpu(), d["qweight"], d["scales"], d["qzeros"], 128)
    with pytest.raises(ValueError):
        ops_mod.int4_gemv(d["x"], d["qweight"], d["scales"], d["qzeros"], 96)
    with pytest.raises(ValueError):
        ops_mod.int4_gemv(d["x"].t().contiguous().t(), d["qweight"], d["scales"], d["qzeros"], 128)


# ------------------------------------------------------------------ plan-free launches of prepacked weights
DIRECT_SHAPES = [
    # M, K, N, fused
    (1, 2048, 2048, False), (1, 5632, 2048, False), (1, 2048, 5632, False), (1, 11008, 96, False),
    (1, 128, 16, False), (3, 640, 50, False), (16, 1536, 64, False), (7, 4096, 80, False),
    (1, 2048, 2 * 5632, True), (8, 2048, 2 * 704, True), (5, 4096, 2 * 48, True),
    # more than one slab of rows, several tiles per workgroup, a ragged last workgroup
    (32, 2048, 2048, False), (17, 2048, 100, False), (32, 5632, 208, False), (9, 1024, 80, False),
    (32, 11008, 48, False), (32, 2048, 2 * 720, True), (20, 4096, 2 * 112, True), (16, 2048, 2064, False),
    # long K with register-fed activations: two super-chunks per wave (ragged share, full share), and more
    # tiles than the device holds workgroups (a workgroup walks two sets)
    (12, 8704, 64, False), (16, 16384, 32, False), (4, 11008, 4352, False), (2, 4096, 2 * 8256, True),
]


@pytest.mark.parametrize("M,K,N,fused", DIRECT_SHAPES)
def test_direct_prepacked_parity(ops_mod, M, K, N, fused):
    say("direct prepacked", M, K, N, fused)
    G = 128
    ops = o.make_operands(9000 + M + K + N, M, K, N, G)
    d = to_device(ops, DEV)
    pw = ops_mod.int4_prepack(d["qweight"], d["scales"], d["qzeros"], G)
    (y,) = ops_mod.DirectGemv([(d["x"], pw, fused)]).launch()
    torch.cuda.synchronize()
    if not fused:
        assert_gemv_close(bf16_to_bits(y), ops, G, f"direct M{M} K{K} N{N}")
        return
    args = (ops["x_bits"], ops["qweight"], ops["scales_bits"], ops["qzeros"], G)
    ref = o.gate_up_silu_f64(*args)
    got = o.bf16_bits_to_f32(bf16_to_bits(y)).astype(np.float64)
    tol = np.maximum(2 * o.bf16_ulp(ref), 1e-2 * np.abs(ref)) + 1e-5
    assert got.shape == ref.shape and (np.abs(got - ref) <= tol).all()


# 17 to 32 rows of K > 2048 with enough tiles: activations staged in passes over K, either one record for all the
# rows (K up to 4096, 512 tiles or more) or records of 16 rows with eight waves per tile (256 tiles or more)
ROWS32_SHAPES = [
    # M, K, N, fused, G
    (32, 4096, 8192, False, 128), (17, 2560, 8200, False, 128), (24, 4096, 2 * 8192, True, 128),
    (32, 3072, 8192, False, 64), (32, 4096, 2 * 8192, True, 32),
    (32, 11008, 4096, False, 128), (20, 4096, 4100, False, 128), (32, 8704, 4096, False, 64),
    (31, 4608, 4096, False, 32),
]


@pytest.mark.parametrize("M,K,N,fused,G", ROWS32_SHAPES)
def test_direct_prepacked_parity_rows_17_to_32_long_k(ops_mod, M, K, N, fused, G):
    say("direct prepacked, passes over K", M, K, N, fused, G)
    ops = o.make_operands(9400 + M + K + N + G, M, K, N, G)
    d = to_device(ops, DEV)
    pw = ops_mod.int4_prepack(d["qweight"], d["scales"], d["qzeros"], G)
    (y,) = ops_mod.DirectGemv([(d["x"], pw, fused)]).launch()
    torch.cuda.synchronize()
    if not fused:
        assert_gemv_close(bf16_to_bits(y), ops, G, f"direct M{M} K{K} N{N} G{G}")
        # rows do not depend on how many travel together: the first rows alone take the 16-row forms
        (y8,) = ops_mod.DirectGemv([(d["x"][:8].contiguous(), pw, False)]).launch()
        torch.cuda.synchronize()
        assert_gemv_close(bf16_to_bits(y8), {**ops, "x_bits": ops["x_bits"][:8]}, G, "first rows alone")
        return
    assert_gate_up_close(bf16_to_bits(y), ops, G, f"direct fused M{M} K{K} N{N} G{G}")


def test_direct_rows32_group_of_three_and_one_hot(ops_mod):
    """A q|k|v-like group at 32 rows of K = 4096 (one record per problem for all rows): each output against the
    oracle, and one-hot activations return the exact weight columns in both row blocks."""
    say("direct group, 32 rows")
    G, M, K = 128, 32, 4096
    probs, checks = [], []
    for i, N in enumerate((4096, 4096, 1024)):
        ops = o.make_operands(9500 + i, M, K, N, G)
        d = to_device(ops, DEV)
        if i:
            d["x"] = probs[0][0]
            ops = {**ops, "x_bits": checks[0]["x_bits"]}
        probs.append((d["x"], ops_mod.int4_prepack(d["qweight"], d["scales"], d["qzeros"], G), False))
        checks.append(ops)
    outs = [y.clone() for y in ops_mod.DirectGemv(probs).launch()]
    torch.cuda.synchronize()
    for y, ops in zip(outs, checks):
        assert_gemv_close(bf16_to_bits(y), ops, G, "direct group, 32 rows")
    ops = o.make_operands(9510, M, K, 8192, G, "loguniform")
    w = o.dequant_bf16(ops["qweight"], ops["scales_bits"], ops["qzeros"], G)
    d = to_device(ops, DEV)
    pw = ops_mod.int4_prepack(d["qweight"], d["scales"], d["qzeros"], G)
    x = np.zeros((M, K), dtype=np.float32)
    ks = [(131 * m + 7) % K for m in range(M)]
    for m in range(M):
        x[m, ks[m]] = 1.0
    (y,) = ops_mod.DirectGemv([(bits_to_bf16(o.f32_to_bf16_bits(x), DEV), pw, False)]).launch()
    torch.cuda.synchronize()
    y = bf16_to_bits(y)
    for m in range(M):
        want = w[:, ks[m]]
        assert ((y[m] == want) | (((y[m] | want) & 0x7FFF) == 0)).all(), m


def test_direct_group_matches_single_launches_and_plan(ops_mod):
    """q|k|v-like group of three in one plan-free launch: same bits as one launch each and as a plan."""
    say("direct group")
    G = 128
    probs, checks = [], []
    for i, (M, K, N) in enumerate([(1, 2048, 2048), (1, 2048, 512), (1, 2048, 100)]):
        ops = o.make_operands(9100 + i, M, K, N, G)
        d = to_device(ops, DEV)
        probs.append((d["x"], ops_mod.int4_prepack(d["qweight"], d["scales"], d["qzeros"], G), False))
        checks.append(ops)
    outs = [y.clone() for y in ops_mod.DirectGemv(probs).launch()]
    torch.cuda.synchronize()
    for y, ops in zip(outs, checks):
        assert_gemv_close(bf16_to_bits(y), ops, G, "direct group")
    singles = [ops_mod.DirectGemv([p]).launch()[0] for p in probs]
    planned = ops_mod.GroupedGemv(probs).launch()
    torch.cuda.synchronize()
    for a, b, c in zip(outs, singles, planned):
        assert torch.equal(a, b) and torch.equal(a, c)   # same kernel body, same summation order


def test_direct_one_hot_is_the_exact_weight_column(ops_mod):
    say("direct one-hot")
    G, M, K, N = 128, 2, 1024, 48
    ops = o.make_operands(9200, M, K, N, G, "loguniform")
    w = o.dequant_bf16(ops["qweight"], ops["scales_bits"], ops["qzeros"], G)
    d = to_device(ops, DEV)
    pw = ops_mod.int4_prepack(d["qweight"], d["scales"], d["qzeros"], G)
    for k0 in (0, 5, 127, 128, 511, 512, 777, K - 1):
        x = np.zeros((M, K), dtype=np.float32)
        for m in range(M):
            x[m, (k0 + 300 * m) % K] = 1.0
        (y,) = ops_mod.DirectGemv([(bits_to_bf16(o.f32_to_bf16_bits(x), DEV), pw, False)]).launch()
        torch.cuda.synchronize()
        y = bf16_to_bits(y)
        for m in range(M):
            want = w[:, (k0 + 300 * m) % K]
            assert ((y[m] == want) | (((y[m] | want) & 0x7FFF) == 0)).all(), (k0, m)


def test_direct_rejects_what_it_cannot_take(ops_mod):
    G = 128
    ops = o.make_operands(9300, 33, 256, 32, G)
    d = to_device(ops, DEV)
    pw = ops_mod.int4_prepack(d["qweight"], d["scales"], d["qzeros"], G)
    with pytest.raises(ValueError):
        ops_mod.DirectGemv([(d["x"], pw, False)])            # 33 rows
    with pytest.raises(ValueError):
        ops_mod.DirectGemv([(d["x"][:1], pw, False)] * 9)    # nine problems
    big = o.make_operands(9301, 32, 11008, 16, G)            # two 16-row slabs per problem, eight per launch
    db = to_device(big, DEV)
    pwb = ops_mod.int4_prepack(db["qweight"], db["scales"], db["qzeros"], G)
    assert pwb.direct_slab_rows() == 6                       # the staged form's bound (what LDS holds of such rows)
    ops_mod.DirectGemv([(db["x"], pwb, False)] * 4).launch()
    with pytest.raises(ValueError):
        ops_mod.DirectGemv([(db["x"], pwb, False)] * 5).launch()
