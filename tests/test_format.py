"""Host-side format code of the package against the oracle (CPU only)."""

import numpy as np
import pytest
import torch

from oracle import int4_oracle as o
from tests._util import bf16_to_bits, bits_to_bf16
from visionrl_amd import int4_format as f


def test_pack_known_answer_and_round_trip():
    assert int(f.pack_nibbles(torch.arange(8))[0]) == 0x76543210
    assert int(f.pack_nibbles(torch.arange(8, 16))[0]) & 0xFFFFFFFF == 0xFEDCBA98
    g = torch.Generator().manual_seed(0)
    for shape in [(4, 64), (3, 5, 24), (2, 13)]:
        q = torch.randint(0, 16, shape, generator=g)
        packed = f.pack_nibbles(q)
        assert packed.dtype == torch.int32
        assert torch.equal(f.unpack_nibbles(packed, shape[-1]), q.to(torch.uint8))
        assert (packed.numpy() == o.pack_nibbles(q.numpy())).all()
    with pytest.raises(ValueError):
        f.pack_nibbles(torch.tensor([16]))
    with pytest.raises(TypeError):
        f.pack_nibbles(torch.tensor([1.0]))


def test_check_packed_contract():
    ops = o.make_operands(1, 1, 256, 8, 64)
    qw, sc, qz = (torch.from_numpy(ops["qweight"]), bits_to_bf16(ops["scales_bits"]),
                  torch.from_numpy(ops["qzeros"]))
    assert f.check_packed(qw, sc, qz, 64) == (8, 256, 4)
    with pytest.raises(ValueError):
        f.check_packed(qw, sc, qz, 12)
    with pytest.raises(ValueError):
        f.check_packed(qw, sc[:, :2], qz, 64)
    with pytest.raises(TypeError):
        f.check_packed(qw, sc.float(), qz, 64)
    with pytest.raises(TypeError):
        f.check_packed(qw.long(), sc, qz, 64)
    with pytest.raises(ValueError):
        f.check_packed(qw, sc, torch.zeros(8, 2, dtype=torch.int32), 64)


def test_quantizer_matches_oracle_bit_for_bit():
    g = torch.Generator().manual_seed(2)
    w = torch.randn(12, 384, generator=g) * 0.05
    w[3, :128] = 0.0            # an all-zero group
    w[5, 128:256] = 0.25        # a constant group
    for G in (32, 64, 128):
        qweight, scales, qzeros = f.quantize_minmax(w.to(torch.bfloat16), G)
        q, s_bits, z = o.quantize_minmax(w.to(torch.bfloat16).float().numpy(), G)
        assert (qweight.numpy() == o.pack_nibbles(q)).all()
        assert (bf16_to_bits(scales) == s_bits).all()
        assert (qzeros.numpy() == o.pack_nibbles(z)).all()
        f.check_packed(qweight, scales, qzeros, G)


def test_algorithmic_bytes_agree():
    for args in [(1, 2048, 2048, 128), (32, 2048, 16384, 128), (8, 4096, 22016, 128)]:
        assert f.algorithmic_bytes(*args) == o.algorithmic_bytes(*args)
    assert f.algorithmic_bytes(8, 4096, 22016, 128, True) == 47_091_712
