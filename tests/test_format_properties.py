"""Property tests of the packed format and quantiser (CPU, hypothesis)."""

import numpy as np
import torch
from hypothesis import given, settings, strategies as st

from oracle import int4_oracle as o
from visionrl_amd import int4_format as f


@settings(max_examples=60, deadline=None)
@given(st.integers(1, 5), st.integers(1, 70), st.integers(0, 2 ** 31 - 1))
def test_pack_round_trip_any_length(rows, length, seed):
    q = np.random.default_rng(seed).integers(0, 16, (rows, length), dtype=np.uint8)
    packed = f.pack_nibbles(torch.from_numpy(q.astype(np.int64)))
    assert packed.shape == (rows, (length + 7) // 8)
    assert (packed.numpy() == o.pack_nibbles(q)).all()
    assert (f.unpack_nibbles(packed, length).numpy() == q).all()
    # padding nibbles are zero
    full = f.unpack_nibbles(packed, packed.shape[-1] * 8).numpy()
    assert (full[:, length:] == 0).all()


@settings(max_examples=40, deadline=None)
@given(st.sampled_from([8, 16, 32, 64, 128]), st.integers(1, 4), st.integers(1, 6),
       st.floats(1e-4, 10.0), st.integers(0, 2 ** 31 - 1))
def test_quantiser_invariants(G, groups, rows, spread, seed):
    rng = np.random.default_rng(seed)
    w = (rng.normal(0, spread, (rows, G * groups))).astype(np.float32)
    qweight, scales, qzeros = f.quantize_minmax(torch.from_numpy(w), G)
    N, K, ng = f.check_packed(qweight, scales, qzeros, G)
    assert (N, K, ng) == (rows, G * groups, groups)
    q = f.unpack_nibbles(qweight, K).numpy().astype(np.float32)
    z = f.unpack_nibbles(qzeros, ng).numpy().astype(np.float32)
    s = scales.float().numpy()
    assert (s > 0).all()
    deq = (q.reshape(rows, ng, G) - z[:, :, None]) * s[:, :, None]
    err = np.abs(deq.reshape(rows, K) - w).reshape(rows, ng, G)
    assert (err <= 1.02 * s[:, :, None]).all()
    # the oracle's quantiser and the package's agree bit for bit
    q2, s2, z2 = o.quantize_minmax(w, G)
    assert (q2 == q.astype(np.uint8)).all() and (z2 == z.astype(np.uint8)).all()
    assert (s2 == scales.view(torch.int16).numpy().view(np.uint16)).all()
    # and the canonical tile of the packed result is what the closed form says
    tile = o.bf16_bits_to_f32(o.dequant_bf16(qweight.numpy(), s2, qzeros.numpy(), G))
    want = torch.from_numpy(deq.reshape(rows, K).astype(np.float32)).to(torch.bfloat16).float().numpy()
    assert (tile == want).all()
