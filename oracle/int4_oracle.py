"""CPU oracle for the int4 weight-only decode linears.  TEST INFRASTRUCTURE ONLY.

Nothing in the shipped package may import this module: it is the checker that
tests, the smoke run and the benchmark's CPU-baseline leg use, never the thing
measured or shipped.

What it restates.  The reference (guoriyue/VisionRL) runs its decode-time
linears as third-party bf16 ``nn.Linear`` modules
(``vrl/models/families/janus_pro/policy.py:673-678`` calls the Llama trunk,
``policy.py:138-160`` calls ``gen_head``); it contains no quantised operator, no
packed-weight format and no numeric golden vector for this path
(``tests/models/test_janus_wrapper.py:30-87`` replaces the trunk by an identity
stub).  The int4 contract below is therefore the closed form the benchmark
configuration states: weights uint4 packed 8 per int32 along K, one bf16 scale
and one uint4 zero-point per group of ``G`` consecutive k, bf16 activations,
fp32 accumulation, bf16 output:

    w[n,k] = bf16_rne( fp32(q[n,k] - z[n,k//G]) * fp32(s[n,k//G]) )
    y[m,n] = bf16_rne( sum_k fp32(x[m,k]) * w[n,k] )

Parity status.  Against the reference: PARITY UNPINNED for every function
(the reference holds nothing to compare with).  Each function is instead pinned
by mathematics in ``tests/test_oracle.py``: known-answer words, exhaustive
(q, z) x scale sweeps evaluated with exact integer/rational arithmetic,
``torch.Tensor.to(bfloat16)`` as the library rounding routine, special cases
that reduce the GEMV to an integer matmul or to a column of the dequant tile,
and the independent C restatement in ``int4_oracle.c``.

``cfg_sample`` restates the tensor ops that follow the image-token head in a decode step
(``policy.py:686-693``).  Their arithmetic lives in torch, not in the reference; the function is
pinned (``tests/test_cfg_sample.py``) by closed forms (constant noise samples the mode of the
guided logits evaluated independently in float64, zero guidance weight ignores the conditional
rows, the log-probability against a float64 log-softmax, a tiny draw wins), and by running the
very same torch ops in bfloat16: on the CPU for temperatures where dividing and multiplying by
the reciprocal coincide, and on the device (GPU tests) under one seed for the rest.  The
reference's tests hold no numeric vector for it (``tests/models/test_janus_wrapper.py:142-175``
checks shapes, dtypes and ranges only): PARITY UNPINNED against the reference here too.

bf16 values travel as ``uint16`` bit patterns (numpy has no bf16 dtype).
"""

from __future__ import annotations

import numpy as np

NIBBLES_PER_WORD = 8


# --------------------------------------------------------------------------
# bf16 <-> fp32 on bit patterns
# --------------------------------------------------------------------------

def bf16_bits_to_f32(bits: np.ndarray) -> np.ndarray:
    """uint16 bf16 bit patterns -> float32 (exact: bf16 is the top half of fp32)."""
    bits = np.asarray(bits, dtype=np.uint16)
    return (bits.astype(np.uint32) << np.uint32(16)).view(np.float32)


def f32_to_bf16_bits(values: np.ndarray) -> np.ndarray:
    """float32 -> bf16 bit patterns, round-to-nearest-even.

    The textbook integer form: add 0x7FFF plus the lsb that survives, then
    truncate.  NaN keeps a quiet payload bit so it stays NaN after truncation.
    """
    v = np.ascontiguousarray(values, dtype=np.float32)
    u = v.view(np.uint32)
    lsb = (u >> np.uint32(16)) & np.uint32(1)
    rounded = (u + np.uint32(0x7FFF) + lsb) >> np.uint32(16)
    is_nan = np.isnan(v)
    nan_bits = (u >> np.uint32(16)) | np.uint32(0x0040)
    return np.where(is_nan, nan_bits, rounded).astype(np.uint16)


def bf16_ulp(values: np.ndarray) -> np.ndarray:
    """Spacing of bf16 numbers at |values| (float64 in, float64 out).

    bf16 has 8 significant bits, so ulp = 2**(floor(log2|v|) - 7); below the
    smallest normal the spacing is the subnormal step 2**-133.
    """
    a = np.abs(np.asarray(values, dtype=np.float64))
    e = np.floor(np.log2(np.maximum(a, 2.0 ** -126)))
    return np.exp2(e - 7.0)


# --------------------------------------------------------------------------
# packing
# --------------------------------------------------------------------------

def pack_nibbles(q: np.ndarray) -> np.ndarray:
    """uint4 values [..., L] -> int32 [..., ceil(L/8)].

    Nibble i (bits 4i..4i+3) of word r holds q[..., 8r+i]; the last word is
    zero-padded.  Known answer: q = 0,1,...,7 packs to 0x76543210.
    """
    q = np.asarray(q)
    if q.size and (q.min() < 0 or q.max() > 15):
        raise ValueError("nibble values must lie in [0, 15]")
    L = q.shape[-1]
    words = (L + NIBBLES_PER_WORD - 1) // NIBBLES_PER_WORD
    padded = np.zeros(q.shape[:-1] + (words * NIBBLES_PER_WORD,), dtype=np.uint32)
    padded[..., :L] = q
    padded = padded.reshape(q.shape[:-1] + (words, NIBBLES_PER_WORD))
    shifts = (np.arange(NIBBLES_PER_WORD, dtype=np.uint32) * np.uint32(4))
    packed = np.bitwise_or.reduce(padded << shifts, axis=-1).astype(np.uint32)
    return packed.view(np.int32)


def unpack_nibbles(packed: np.ndarray, length: int) -> np.ndarray:
    """int32 [..., W] -> uint8 [..., length]; inverse of :func:`pack_nibbles`."""
    u = np.ascontiguousarray(packed, dtype=np.int32).view(np.uint32)
    shifts = (np.arange(NIBBLES_PER_WORD, dtype=np.uint32) * np.uint32(4))
    nib = (u[..., None] >> shifts) & np.uint32(0xF)
    nib = nib.reshape(u.shape[:-1] + (u.shape[-1] * NIBBLES_PER_WORD,))
    if length > nib.shape[-1]:
        raise ValueError("length exceeds packed capacity")
    return nib[..., :length].astype(np.uint8)


def check_shapes(qweight, scales, qzeros, group_size):
    """Validate the packed operand triple; returns (N, K, groups)."""
    if qweight.ndim != 2 or scales.ndim != 2 or qzeros.ndim != 2:
        raise ValueError("qweight, scales and qzeros must be 2-D")
    N, kw = qweight.shape
    K = kw * NIBBLES_PER_WORD
    G = int(group_size)
    if G <= 0 or G % NIBBLES_PER_WORD != 0:
        raise ValueError("group_size must be a positive multiple of 8")
    if K % G != 0:
        raise ValueError("K must be a multiple of group_size")
    groups = K // G
    if scales.shape != (N, groups):
        raise ValueError(f"scales must be [{N}, {groups}]")
    zw = (groups + NIBBLES_PER_WORD - 1) // NIBBLES_PER_WORD
    if qzeros.shape != (N, zw):
        raise ValueError(f"qzeros must be [{N}, {zw}]")
    return N, K, groups


# --------------------------------------------------------------------------
# dequant and GEMV
# --------------------------------------------------------------------------

def dequant_bf16(qweight, scales_bits, qzeros, group_size) -> np.ndarray:
    """Packed int4 -> bf16 bit patterns [N, K] (the canonical weight tile).

    The fp32 product (q - z) * s is exact (|q - z| <= 15 needs 4 bits, a bf16
    scale has 8 significant bits, so the product has at most 12), hence the only
    rounding is the final round-to-nearest-even to bf16.
    """
    N, K, groups = check_shapes(qweight, scales_bits, qzeros, group_size)
    q = unpack_nibbles(qweight, K).astype(np.int32)
    z = unpack_nibbles(qzeros, groups).astype(np.int32)
    s = bf16_bits_to_f32(scales_bits)
    d = (q.reshape(N, groups, group_size) - z[:, :, None]).astype(np.float32)
    w = d * s[:, :, None]
    return f32_to_bf16_bits(w.reshape(N, K))


def gemv_f64(x_bits, qweight, scales_bits, qzeros, group_size) -> np.ndarray:
    """Truth for the GEMV: float64 ``x @ w.T`` over the canonical bf16 weights.

    Returns float64 [M, N]; no output rounding.  Products of two bf16 numbers
    are exact in float64 and K <= 2**20 such products sum with relative error
    far below fp32 resolution.
    """
    w = bf16_bits_to_f32(dequant_bf16(qweight, scales_bits, qzeros, group_size))
    x = bf16_bits_to_f32(np.asarray(x_bits, dtype=np.uint16))
    return x.astype(np.float64) @ w.astype(np.float64).T


def gemv_abs_f64(x_bits, qweight, scales_bits, qzeros, group_size) -> np.ndarray:
    """sum_k |x[m,k] * w[n,k]| in float64: the scale of fp32 accumulation noise."""
    w = bf16_bits_to_f32(dequant_bf16(qweight, scales_bits, qzeros, group_size))
    x = bf16_bits_to_f32(np.asarray(x_bits, dtype=np.uint16))
    return np.abs(x).astype(np.float64) @ np.abs(w).astype(np.float64).T


def gemv_and_abs_f64(x_bits, qweight, scales_bits, qzeros, group_size):
    """``(gemv_f64, gemv_abs_f64)`` of one operand set over one dequantisation (large matrices)."""
    w = bf16_bits_to_f32(dequant_bf16(qweight, scales_bits, qzeros, group_size)).astype(np.float64)
    x = bf16_bits_to_f32(np.asarray(x_bits, dtype=np.uint16)).astype(np.float64)
    return x @ w.T, np.abs(x) @ np.abs(w).T


def gemv_bf16(x_bits, qweight, scales_bits, qzeros, group_size) -> np.ndarray:
    """The operator itself: fp32 accumulate (numpy pairwise order), bf16 out."""
    w = bf16_bits_to_f32(dequant_bf16(qweight, scales_bits, qzeros, group_size))
    x = bf16_bits_to_f32(np.asarray(x_bits, dtype=np.uint16))
    return f32_to_bf16_bits((x @ w.T).astype(np.float32))


def silu_f64(v: np.ndarray) -> np.ndarray:
    v = np.asarray(v, dtype=np.float64)
    return v / (1.0 + np.exp(-v))


def gate_up_silu_f64(x_bits, qweight_gu, scales_gu, qzeros_gu, group_size) -> np.ndarray:
    """Truth for the fused MLP front half: SiLU(x Wg^T) * (x Wu^T) in float64.

    Rows 0..I-1 of the packed operand are the gate projection, rows I..2I-1 the
    up projection (the order ``LlamaMLP`` applies them: act(gate(x)) * up(x)).
    """
    acc = gemv_f64(x_bits, qweight_gu, scales_gu, qzeros_gu, group_size)
    inter = acc.shape[1] // 2
    if acc.shape[1] != 2 * inter:
        raise ValueError("gate||up operand needs an even number of rows")
    return silu_f64(acc[:, :inter]) * acc[:, inter:]


def gate_up_silu_bf16(x_bits, qweight_gu, scales_gu, qzeros_gu, group_size) -> np.ndarray:
    """Fused operator: fp32 accumulators, fp32 SiLU and product, one bf16 rounding."""
    w = bf16_bits_to_f32(dequant_bf16(qweight_gu, scales_gu, qzeros_gu, group_size))
    x = bf16_bits_to_f32(np.asarray(x_bits, dtype=np.uint16))
    acc = (x @ w.T).astype(np.float32)
    inter = acc.shape[1] // 2
    g, u = acc[:, :inter], acc[:, inter:]
    act = (g / (np.float32(1.0) + np.exp(-g, dtype=np.float32))).astype(np.float32)
    return f32_to_bf16_bits(act * u)


# an output counts as cancelled when it is this small against the sum of its terms' magnitudes
CANCELLED_BELOW = 2.0 ** -6
# fp32 reassociation noise allowed on a cancelled output, as a fraction of sum|x w|
CANCELLED_SLACK = 2.0 ** -18


def gemv_strict_tolerance(y_ref: np.ndarray) -> np.ndarray:
    """The stated operator tolerance: max(1 bf16 ulp at y_ref, 1e-2 * |y_ref|)."""
    y_ref = np.asarray(y_ref, dtype=np.float64)
    return np.maximum(bf16_ulp(y_ref), 1e-2 * np.abs(y_ref))


def gemv_cancelled(y_ref: np.ndarray, abs_ref: np.ndarray) -> np.ndarray:
    """Outputs whose terms cancel: |y_ref| < 2**-6 * sum|x w|."""
    return np.abs(np.asarray(y_ref, dtype=np.float64)) < CANCELLED_BELOW * np.asarray(abs_ref, dtype=np.float64)


def gemv_tolerance(y_ref: np.ndarray, abs_ref: np.ndarray) -> np.ndarray:
    """Allowed |y - y_ref| per element for a bf16 output with fp32 accumulation.

    The stated tolerance max(1 bf16 ulp at y_ref, 1e-2 * |y_ref|) holds as it is for every output
    with |y_ref| >= 2**-6 * sum|x w|.  Outputs that cancel further than that (a relative bound on
    a sum that is almost zero says nothing about the summation) may carry the reassociation noise
    of an fp32 accumulation in any order on top: 2**-18 * sum|x w|.
    """
    strict = gemv_strict_tolerance(y_ref)
    return np.where(gemv_cancelled(y_ref, abs_ref), strict + CANCELLED_SLACK * np.asarray(abs_ref, np.float64), strict)


# --------------------------------------------------------------------------
# quantiser (loader glue restated)
# --------------------------------------------------------------------------

def quantize_minmax(w: np.ndarray, group_size: int):
    """Asymmetric min/max uint4 quantiser, one (scale, zero) per K-group.

    s = bf16((max - min) / 15) (1 if the group is constant), z = clamp(rne(-min/s)),
    q = clamp(rne(w / s) + z, 0, 15), all in float32 with the bf16-rounded scale.
    Returns (q uint8 [N,K], scales_bits uint16 [N,K/G], z uint8 [N,K/G]).
    """
    w = np.asarray(w, dtype=np.float32)
    N, K = w.shape
    G = int(group_size)
    if K % G != 0:
        raise ValueError("K must be a multiple of group_size")
    g = w.reshape(N, K // G, G)
    lo = np.minimum(g.min(axis=-1), np.float32(0.0))
    hi = np.maximum(g.max(axis=-1), np.float32(0.0))
    span = (hi - lo).astype(np.float32)
    raw = np.where(span > 0, span / np.float32(15.0), np.float32(1.0)).astype(np.float32)
    s_bits = f32_to_bf16_bits(raw)
    s = bf16_bits_to_f32(s_bits)
    z = np.clip(np.rint(-lo / s), 0, 15).astype(np.float32)
    q = np.clip(np.rint(g / s[:, :, None]) + z[:, :, None], 0, 15)
    return q.reshape(N, K).astype(np.uint8), s_bits, z.astype(np.uint8)


# --------------------------------------------------------------------------
# seeded synthetic operands (benchmark configurations)
# --------------------------------------------------------------------------

def make_operands(seed: int, M: int, K: int, N: int, G: int, scale_mode: str = "normal"):
    """Seeded operands with the benchmark's value distributions.

    q, z ~ U{0..15}; s = |N(0, 0.02)| as bf16 (``normal``, exact zeros resampled
    to the smallest drawn positive value) or 10**U(-4,-1) as bf16
    (``loguniform``); x ~ N(0,1) as bf16.  Returns a dict of numpy arrays:
    x_bits [M,K] u16, qweight [N,K/8] i32, scales_bits [N,K/G] u16,
    qzeros [N,ceil(K/G/8)] i32, plus unpacked q and z.
    """
    rng = np.random.default_rng(seed)
    groups = K // G
    q = rng.integers(0, 16, size=(N, K), dtype=np.uint8)
    z = rng.integers(0, 16, size=(N, groups), dtype=np.uint8)
    if scale_mode == "normal":
        s = np.abs(rng.normal(0.0, 0.02, size=(N, groups))).astype(np.float32)
    elif scale_mode == "loguniform":
        s = np.power(10.0, rng.uniform(-4.0, -1.0, size=(N, groups))).astype(np.float32)
    else:
        raise ValueError(f"unknown scale_mode {scale_mode!r}")
    s_bits = f32_to_bf16_bits(s)
    if (s_bits == 0).any():
        s_bits[s_bits == 0] = s_bits[s_bits != 0].min()
    x = rng.normal(0.0, 1.0, size=(M, K)).astype(np.float32)
    return {
        "x_bits": f32_to_bf16_bits(x),
        "qweight": pack_nibbles(q),
        "scales_bits": s_bits,
        "qzeros": pack_nibbles(z),
        "q": q,
        "z": z,
    }


def algorithmic_bytes(M: int, K: int, N: int, G: int, fused_gate_up: bool = False) -> int:
    """4-bit weights + bf16 scales + 4-bit zeros + bf16 x + bf16 y, in bytes.

    For the fused gate||up operator N counts both halves for the reads and the
    output has N/2 columns.
    """
    groups = K // G
    out_cols = N // 2 if fused_gate_up else N
    return K * N // 2 + groups * N * 2 + groups * N // 2 + M * K * 2 + M * out_cols * 2


# --------------------------------------------------------------------------
# the CPU path a user of the reference would run: PyTorch dequant + matmul
# --------------------------------------------------------------------------

def torch_dequant(qweight, scales, qzeros, group_size):
    """``((q - z).float() * s.float()).to(bfloat16)`` on torch CPU tensors."""
    import torch

    N, kw = qweight.shape
    K = kw * NIBBLES_PER_WORD
    groups = K // group_size
    shifts = torch.arange(0, 32, 4, dtype=torch.int32)
    q = ((qweight.unsqueeze(-1) >> shifts) & 0xF).reshape(N, K)
    z = ((qzeros.unsqueeze(-1) >> shifts) & 0xF).reshape(N, -1)[:, :groups]
    d = (q.reshape(N, groups, group_size) - z.unsqueeze(-1)).float()
    return (d * scales.float().unsqueeze(-1)).to(torch.bfloat16).reshape(N, K)


def torch_cpu_linear(x, qweight, scales, qzeros, group_size):
    """Dequantise then ``torch.nn.functional.linear`` in bf16 (the CPU baseline)."""
    import torch

    return torch.nn.functional.linear(x, torch_dequant(qweight, scales, qzeros, group_size))


# ---------------------------------------------------------------------------
# decode-step tail: CFG combine, softmax, one multinomial draw, log-probability
# Follows vrl/models/families/janus_pro/policy.py:686-693 with the arithmetic torch applies
# to bf16 tensors (fp32 per op, result rounded to bf16; tensor / host scalar is a product
# with fl(1/scalar); multinomial(probs, 1) is argmax(probs / q), q ~ Exp(1)).
# ---------------------------------------------------------------------------
def _round_bf16_f32(v: np.ndarray) -> np.ndarray:
    return bf16_bits_to_f32(f32_to_bf16_bits(np.asarray(v, dtype=np.float32)))


def cfg_sample(logits_bits: np.ndarray, noise_bits: np.ndarray, cfg_weight: float, temperature: float):
    """Returns ``(sampled [B] int64, logprob [B] float32, probs [B,V] float32, ratio [B,V] float32)``.

    ``logits_bits`` uint16 ``[2B, V]`` (conditional rows first), ``noise_bits`` uint16 ``[B, V]``.
    ``probs`` and ``ratio`` (= probs / noise, the quantity whose argmax is the draw) are
    returned so that a test can judge near-ties.
    """
    f32 = np.float32
    B = logits_bits.shape[0] // 2
    c = bf16_bits_to_f32(logits_bits[:B])
    u = bf16_bits_to_f32(logits_bits[B:])
    q = bf16_bits_to_f32(noise_bits)
    w, inv_t = f32(cfg_weight), f32(1.0) / f32(temperature)
    d = _round_bf16_f32(c - u)
    g = _round_bf16_f32(u + _round_bf16_f32(w * d))
    gt = _round_bf16_f32(g * inv_t)
    ct = _round_bf16_f32(c * inv_t)
    eg = np.exp((gt - gt.max(axis=1, keepdims=True)).astype(f32)).astype(f32)
    probs = _round_bf16_f32(eg / eg.sum(axis=1, keepdims=True, dtype=f32))
    with np.errstate(divide="ignore", invalid="ignore"):
        ratio = _round_bf16_f32(probs / q)
    sampled = np.argmax(ratio, axis=1).astype(np.int64)          # first index among equal maxima
    mc = ct.max(axis=1, keepdims=True)
    lse = np.log(np.exp((ct - mc).astype(f32)).astype(f32).sum(axis=1, keepdims=True, dtype=f32)).astype(f32)
    lp_all = _round_bf16_f32(ct - mc - lse)
    logprob = lp_all[np.arange(B), sampled].astype(f32)
    return sampled, logprob, probs, ratio
