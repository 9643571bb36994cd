"""The allocation-free head + sampling entry point (``vrl_int4_head_sample_static_bf16``) against the
entry point it is a variant of (``vrl_int4_head_sample_bf16``, caller's workspace), through the C ABI.

Two calls in a row over the library's one scratch array, the second with a smaller input (fewer rows, a
shorter vocabulary): what the first call left in the array must not leak into the second.  Outputs are
compared bit for bit: both entry points run the same kernel, only the scratch memory differs.
"""

import ctypes

import numpy as np
import pytest
import torch

from oracle import int4_oracle as o
from tests._util import bits_to_bf16, to_device
from tests.test_cfg_sample import check_against_oracle
from tests.test_head_sample import make_head

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def call_both(lib, _lib, ops, B, K, V, G, seed, w=5.0, T=1.0):
    operands, nb = make_head(seed, B, K, V, G)
    d = to_device(operands, DEV)
    pw = ops.int4_prepack(d["qweight"], d["scales"], d["qzeros"], G)
    noise = bits_to_bf16(nb, DEV)
    logits = torch.empty((2 * B, V), dtype=torch.bfloat16, device=DEV)
    rec = _lib.Problem()
    rec.x, rec.qweight, rec.y = d["x"].data_ptr(), pw.blob.data_ptr(), logits.data_ptr()
    rec.M, rec.N, rec.K, rec.G, rec.prepacked = 2 * B, V, K, G, 1
    stream = torch.cuda.current_stream().cuda_stream
    ws = ops.head_sample_workspace(B, V, DEV)
    want_s = torch.empty(B, dtype=torch.int64, device=DEV)
    want_lp = torch.empty(B, dtype=torch.float32, device=DEV)
    rc = lib.vrl_int4_head_sample_bf16(ctypes.byref(rec), noise.data_ptr(), want_s.data_ptr(), want_lp.data_ptr(), B,
                                       w, T, ws.data_ptr(), ws.numel(), stream)
    assert rc == 0, _lib.error_string(rc)
    got_s = torch.full((B,), -1, dtype=torch.int64, device=DEV)
    got_lp = torch.full((B,), 7.0, dtype=torch.float32, device=DEV)
    torch.cuda.synchronize()
    before = torch.cuda.memory_allocated()
    rc = lib.vrl_int4_head_sample_static_bf16(ctypes.byref(rec), noise.data_ptr(), got_s.data_ptr(), got_lp.data_ptr(),
                                              B, w, T, stream)
    assert rc == 0, _lib.error_string(rc)
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    assert torch.equal(got_s, want_s) and torch.equal(got_lp, want_lp), (B, V, got_s, want_s, got_lp, want_lp)
    from tests._util import bf16_to_bits
    exact = check_against_oracle(got_s, got_lp, bf16_to_bits(logits), nb, w, T)     # and both are right
    assert exact >= B - max(1, B // 8)
    return rec, noise, got_s, got_lp


def test_static_scratch_entry_point_equals_the_workspace_one():
    from visionrl_amd import _lib, ops

    lib = _lib.load()
    print("[case] no-alloc head_sample: B=16 V=16384, then B=3 V=4096", flush=True)
    call_both(lib, _lib, ops, 16, 2048, 16384, 128, seed=901)          # fills the whole array
    call_both(lib, _lib, ops, 3, 2048, 4096, 128, seed=902)            # smaller: fewer rows, fewer tiles
    call_both(lib, _lib, ops, 16, 2048, 16384, 128, seed=903)          # and the full size again
    # beyond the array: refused with its own code, nothing enqueued
    rec, noise, s, lp = call_both(lib, _lib, ops, 1, 512, 64, 128, seed=904)
    stream = torch.cuda.current_stream().cuda_stream
    rec.N = 16384 + 16
    assert lib.vrl_int4_head_sample_static_bf16(ctypes.byref(rec), noise.data_ptr(), s.data_ptr(), lp.data_ptr(), 1,
                                                5.0, 1.0, stream) == 1005
    rec.N = 64
    assert lib.vrl_int4_head_sample_static_bf16(ctypes.byref(rec), noise.data_ptr(), s.data_ptr(), lp.data_ptr(), 17,
                                                5.0, 1.0, stream) == 1005
    assert "scratch" in _lib.error_string(1005)
    # through the Python surface: the same result as with a workspace tensor, nothing allocated by the call
    operands, nb = make_head(905, 2, 2048, 16384, 128)
    d = to_device(operands, DEV)
    pw = ops.int4_prepack(d["qweight"], d["scales"], d["qzeros"], 128)
    noise = bits_to_bf16(nb, DEV)
    want = ops.head_sample(d["x"], pw, 5.0, 1.0, noise=noise)
    out = (torch.empty(2, dtype=torch.int64, device=DEV), torch.empty(2, dtype=torch.float32, device=DEV))
    torch.cuda.synchronize()
    allocations = lambda: torch.cuda.memory_stats()["allocation.all.allocated"]   # requests served so far
    before = allocations()
    got = ops.head_sample(d["x"], pw, 5.0, 1.0, noise=noise, workspace="static", out=out)
    torch.cuda.synchronize()
    assert allocations() == before and got[0] is out[0]
    assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1])
