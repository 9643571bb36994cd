"""The C-ABI library loads, exports what the header declares and rejects bad calls.

No kernel is launched here: precondition checks run on the host before any HIP
call, so these tests need no GPU.
"""

import ctypes
import os
import re

import pytest

from visionrl_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADERS = [os.path.join(ROOT, "include", name) for name in ("vrl_int4.h", "vrl_decode.h")]


@pytest.fixture(scope="module")
def lib():
    return _lib.load()


def declared_symbols():
    names = set()
    for header in HEADERS:
        text = re.sub(r"/\*.*?\*/", "", open(header).read(), flags=re.S)
        names |= set(re.findall(r"\b(vrl_[a-z0-9_]+)\s*\(", text))
    return sorted(names)


def test_every_declared_symbol_is_exported(lib):
    names = declared_symbols()
    assert set(names) == set(_lib.SYMBOLS)
    for name in names:
        assert hasattr(lib, name), name


def test_abi_version_and_error_strings(lib):
    assert lib.vrl_int4_abi_version() == 1
    assert _lib.error_string(0) == "ok"
    for code in (1001, 1002, 1003, 1004):
        assert "unknown" not in _lib.error_string(code)
    assert "unknown" in _lib.error_string(-5)


def test_problem_struct_matches_header():
    # 5 pointers + 4 ints + flag + 3 reserved ints
    assert ctypes.sizeof(_lib.Problem) == 5 * 8 + 8 * 4


def buf(nbytes, misalign=0):
    raw = ctypes.create_string_buffer(nbytes + 64)
    base = (ctypes.addressof(raw) + 15) & ~15
    return raw, base + misalign


@pytest.mark.parametrize("M,N,K,G,code", [
    (0, 16, 128, 128, 1001),
    (1, 0, 128, 128, 1001),
    (1, 16, 0, 128, 1001),
    (1, 16, 124, 4, 1001),     # K % 8
    (1, 16, 128, 12, 1001),    # G % 8
    (1, 16, 128, 48, 1001),    # K % G
    (1, 16, 128, 0, 1001),
    (-3, 16, 128, 128, 1001),
])
def test_gemv_rejects_bad_shapes(lib, M, N, K, G, code):
    keep, p = buf(4096)
    rc = lib.vrl_int4_gemv_bf16(p, p, p, p, p, M, N, K, G, None)
    assert rc == code
    with pytest.raises(ValueError):
        _lib.check(rc, "gemv")


def test_null_and_alignment_are_reported(lib):
    keep, p = buf(4096)
    assert lib.vrl_int4_gemv_bf16(None, p, p, p, p, 1, 16, 128, 128, None) == 1003
    assert lib.vrl_int4_gemv_bf16(p, p, p, p, None, 1, 16, 128, 128, None) == 1003
    assert lib.vrl_int4_gemv_bf16(p + 2, p, p, p, p, 1, 16, 128, 128, None) == 1002
    assert lib.vrl_int4_gemv_bf16(p, p + 4, p, p, p, 1, 16, 128, 128, None) == 1002
    assert lib.vrl_int4_dequant_bf16(p, p, None, p, 16, 128, 128, None) == 1003
    assert lib.vrl_int4_dequant_bf16(p, p, p, p + 8, 16, 128, 128, None) == 1002
    assert lib.vrl_int4_dequant_bf16(p, p, p, p, 16, 120, 16, None) == 1001
    assert lib.vrl_int4_gate_up_silu_bf16(p, p, p, p, p, 1, 0, 128, 128, None) == 1001
    assert lib.vrl_int4_gate_up_silu_bf16(p, p, p, None, p, 1, 8, 128, 128, None) == 1003


def test_prepacked_size_and_validation(lib):
    keep, p = buf(4096)
    # per 16-row tile: ceil(nsc/4) KiB of scale/zero words + nsc * 4 KiB of weights, nsc = ceil(K/512)
    assert lib.vrl_int4_prepacked_bytes(2048, 2048, 128) == 128 * (4 * 256 + 4 * 4096)
    assert lib.vrl_int4_prepacked_bytes(2048, 5632, 128) == 128 * (11 * 256 + 11 * 4096)
    assert lib.vrl_int4_prepacked_bytes(17, 128, 128) == 2 * (256 + 4096)
    assert lib.vrl_int4_prepacked_bytes(16, 256, 64) == 2 * 256 + 4096    # two meta words per lane
    assert lib.vrl_int4_prepacked_bytes(16, 256, 32) == 4 * 256 + 4096
    assert lib.vrl_int4_prepacked_bytes(16, 256, 16) == 0
    assert lib.vrl_int4_prepacked_bytes(16, 256, 256) == 0
    assert lib.vrl_int4_prepacked_bytes(16, 200, 128) == 0
    assert lib.vrl_int4_prepack(p, p, p, None, 16, 128, 128, None) == 1003
    assert lib.vrl_int4_prepack(p, p, p, p + 4, 16, 128, 128, None) == 1002
    assert lib.vrl_int4_prepack(p, p, p, p, 16, 256, 16, None) == 1001


def test_grouped_plan_validation(lib):
    keep, p = buf(4096)
    assert lib.vrl_int4_grouped_plan_size(0) == 0
    size = lib.vrl_int4_grouped_plan_size(2)
    assert size >= 2 * ctypes.sizeof(_lib.Problem)
    probs = (_lib.Problem * 2)()
    for rec, n in zip(probs, (64, 100)):
        rec.x = rec.qweight = rec.scales = rec.qzeros = rec.y = p
        rec.M, rec.N, rec.K, rec.G = 1, n, 256, 128
    plan = ctypes.create_string_buffer(size)
    info = _lib.PlanInfo()
    assert lib.vrl_int4_grouped_plan_build(probs, 2, plan, size, ctypes.byref(info)) == 0
    assert info.n_problems == 2
    assert info.total_tiles == 4 + 7        # 16-column tiles: 64/16 and ceil(100/16)
    assert 1 <= info.grid <= info.total_tiles and info.block_threads % 64 == 0
    assert info.lds_bytes >= 1 * (256 + 8) * 2
    # the per-workgroup table stored after the records ({first tile, its record} per workgroup)
    # covers every tile exactly once, and names the record each range starts in
    import struct
    rec_bytes = 72   # 5 pointers + 8 int32 per record
    table = struct.unpack_from(f"{2 * (info.grid + 1)}i", plan.raw, 16 + 2 * rec_bytes)
    begins, first_rec = table[0::2], table[1::2]
    assert begins[0] == 0 and begins[-1] == info.total_tiles
    assert all(a <= b for a, b in zip(begins, begins[1:]))
    # records are laid out longest tiles first (equal K here: caller order kept), record 1 starts at tile 4
    assert all(r == (1 if b >= 4 else 0) for b, r in zip(begins, first_rec))
    # undersized buffer, bad shape inside the list, shapes only the generic kernel takes, nulls
    assert lib.vrl_int4_grouped_plan_build(probs, 2, plan, size - 1, ctypes.byref(info)) == 1004
    probs[1].K = 100
    assert lib.vrl_int4_grouped_plan_build(probs, 2, plan, size, ctypes.byref(info)) == 1001
    probs[1].K, probs[1].G = 192, 24
    assert lib.vrl_int4_grouped_plan_build(probs, 2, plan, size, ctypes.byref(info)) == 1001
    assert lib.vrl_int4_grouped_plan_build(None, 2, plan, size, ctypes.byref(info)) == 1003
    assert lib.vrl_int4_gemv_grouped_bf16(None, ctypes.byref(info), None) == 1003
    bad = _lib.PlanInfo()
    assert lib.vrl_int4_gemv_grouped_bf16(p, ctypes.byref(bad), None) == 1004


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", str(tmp_path / "nope.so"))
    with pytest.raises(_lib.Int4LibraryError, match="no CPU or PyTorch fallback"):
        _lib.load()


def test_direct_prepacked_validation(lib):
    keep, p = buf(4096)
    probs = (_lib.Problem * 2)()
    for rec in probs:
        rec.x = rec.qweight = rec.y = p
        rec.M, rec.N, rec.K, rec.G, rec.prepacked = 1, 64, 256, 128, 1
    assert lib.vrl_int4_gemv_prepacked_bf16(None, 1, None) == 1003
    assert lib.vrl_int4_gemv_prepacked_bf16(probs, 0, None) == 1001
    assert lib.vrl_int4_gemv_prepacked_bf16(probs, 9, None) == 1001
    probs[1].prepacked = 0                       # canonical records are not taken here
    assert lib.vrl_int4_gemv_prepacked_bf16(probs, 2, None) == 1001
    probs[1].prepacked, probs[1].M = 1, 16 * 7 + 1   # eight slabs of 16 rows beside the first problem's one
    assert lib.vrl_int4_gemv_prepacked_bf16(probs, 2, None) == 1001
    probs[1].M, probs[1].G = 1, 16               # no prepacked form for this group size
    assert lib.vrl_int4_gemv_prepacked_bf16(probs, 2, None) == 1001
    probs[1].G, probs[1].y = 128, p + 2          # misaligned output
    assert lib.vrl_int4_gemv_prepacked_bf16(probs, 2, None) == 1002
    probs[1].y, probs[1].M, probs[1].K = p, 32, 16896  # beyond the register-fed form; LDS holds 4 such rows: 8 slabs, 9 with the first problem
    assert lib.vrl_int4_gemv_prepacked_bf16(probs, 2, None) == 1001


def test_norm_fused_launch_validation(lib):
    keep, p = buf(1 << 16)
    probs = (_lib.Problem * 2)()
    for rec in probs:
        rec.x = rec.qweight = rec.y = p
        rec.M, rec.N, rec.K, rec.G, rec.prepacked = 1, 64, 256, 128, 1
    norm = _lib.Norm()
    norm.x, norm.weight, norm.eps = p, p, 1e-6
    f = lib.vrl_int4_gemv_prepacked_norm_bf16
    assert f(probs, 2, None, None) == 1003
    norm.weight = None
    assert f(probs, 2, ctypes.byref(norm), None) == 1003
    norm.weight = p
    probs[1].x = p + 512                      # every problem reads the one normalised input
    assert f(probs, 2, ctypes.byref(norm), None) == 1001
    probs[1].x, probs[1].M = p, 2             # ... with the same rows
    assert f(probs, 2, ctypes.byref(norm), None) == 1001
    probs[1].M = 1
    norm.h_out = p                            # h may not overwrite what other workgroups still read
    assert f(probs, 2, ctypes.byref(norm), None) == 1001
    norm.h_out, norm.residual = p + 4096, p + 4096
    assert f(probs, 2, ctypes.byref(norm), None) == 1001
    norm.h_out, norm.residual = None, p + 8
    assert f(probs, 2, ctypes.byref(norm), None) == 1002
    norm.residual, norm.eps = None, -1.0
    assert f(probs, 2, ctypes.byref(norm), None) == 1001
    norm.eps = 1e-6
    for rec in probs:
        rec.K = 8192                          # a row must fit the registers of one wave
    assert f(probs, 2, ctypes.byref(norm), None) == 1001


def test_decode_layer_validation(lib):
    keep, p = buf(1 << 16)
    norm = lib.vrl_add_rmsnorm_bf16
    assert norm(None, None, p, None, p, 1, 256, 1e-6, None) == 1003
    assert norm(p, p, p, None, p, 1, 256, 1e-6, None) == 1003       # a residual needs somewhere to put h
    assert norm(p, None, p, None, p, 0, 256, 1e-6, None) == 1001
    assert norm(p, None, p, None, p, 1, 260, 1e-6, None) == 1001    # K % 8
    assert norm(p, None, p, None, p, 1, 16392, 1e-6, None) == 1001  # K beyond what one workgroup stages
    assert norm(p, None, p, None, p, 1, 256, -1.0, None) == 1001
    assert norm(p + 2, None, p, None, p, 1, 256, 1e-6, None) == 1002
    attn = lib.vrl_rope_attn_decode_bf16
    ok = dict(q=p, k=p, v=p, qs=256, ks=256, kc=p, vc=p, cos=p, sin=p, mask=p, pos=p, out=p,
              M=1, H=4, Hkv=4, D=64, L=16, scale=0.125)

    def call(**over):
        a = dict(ok, **over)
        return attn(a["q"], a["k"], a["v"], a["qs"], a["ks"], a["kc"], a["vc"], a["cos"], a["sin"], a["mask"],
                    a["pos"], a["out"], a["M"], a["H"], a["Hkv"], a["D"], a["L"], a["scale"], None)

    assert call(pos=None) == 1003 and call(mask=None) == 1003
    assert call(D=96) == 1001 and call(Hkv=3) == 1001 and call(L=0) == 1001 and call(L=8193) == 1001
    assert call(qs=128) == 1001          # rows narrower than the heads they hold
    assert call(ks=260) == 1001          # row stride must keep rows 16-byte aligned
    assert call(kc=p + 8) == 1002 and call(pos=p + 4) == 1002
    # the adapter record of the second form
    with_lora = lib.vrl_rope_attn_decode_lora_bf16
    rec = _lib.AttnLora()

    def call_lora(r):
        a = ok
        return with_lora(a["q"], a["k"], a["v"], a["qs"], a["ks"], a["kc"], a["vc"], a["cos"], a["sin"], a["mask"],
                         a["pos"], a["out"], a["M"], a["H"], a["Hkv"], a["D"], a["L"], a["scale"],
                         ctypes.byref(r) if r is not None else None, None)

    assert call_lora(None) == 1003 and call_lora(rec) == 1003     # no record, a record without any adapter
    rec.q_B, rec.r[0], rec.t_stride, rec.weights_fp32 = p, 8, 8, 1
    assert call_lora(rec) == 1003                                 # q/k/v adapters read t
    rec.t, rec.r[0] = p, 12
    assert call_lora(rec) == 1001                                 # rank % 8
    rec.r[0], rec.offset[0] = 8, 4
    assert call_lora(rec) == 1001                                 # the adapter's columns must lie inside a row of t
    rec.offset[0], rec.q_B = 0, None
    rec.o_A, rec.o_r = p, 16
    assert call_lora(rec) == 1003                                 # nowhere to leave the pieces
    rec.o_t, rec.o_r = p, 72
    assert call_lora(rec) == 1001
    rec.o_r, rec.o_t = 16, p + 8
    assert call_lora(rec) == 1002


def test_lora_validation(lib):
    keep, p = buf(1 << 16)
    ads = (_lib.LoraAdapter * 2)()
    for ad in ads:
        ad.A, ad.B, ad.y, ad.N, ad.r, ad.scaling, ad.weights_fp32 = p, p, p, 64, 8, 2.0, 1
    down, up = lib.vrl_lora_down_bf16, lib.vrl_lora_up_add_bf16
    assert down(None, 1, 256, ads, 2, p, None) == 1003 and down(p, 1, 256, None, 2, p, None) == 1003
    assert down(p, 1, 256, ads, 2, None, None) == 1003 and up(None, 1, 1, ads, 2, None) == 1003
    assert down(p, 0, 256, ads, 2, p, None) == 1001 and down(p, 33, 256, ads, 2, p, None) == 1001   # rows
    assert down(p, 1, 260, ads, 2, p, None) == 1001 and down(p, 1, 256, ads, 5, p, None) == 1001    # K % 8, adapters
    ads[1].r = 12
    assert down(p, 1, 256, ads, 2, p, None) == 1001       # rank % 8
    ads[1].r = 72
    assert down(p, 1, 256, ads, 2, p, None) == 1001       # rank beyond 64
    ads[1].r, ads[1].weights_fp32 = 8, 0
    assert down(p, 1, 256, ads, 2, p, None) == 1001       # one weight type per launch
    ads[1].weights_fp32, ads[1].A = 1, p + 8
    assert down(p, 1, 256, ads, 2, p, None) == 1002
    ads[1].A = p
    assert down(p, 1, 256, ads, 2, p + 4, None) == 1002 and up(p + 4, 1, 1, ads, 2, None) == 1002   # t is read 16 bytes at a time
    ads[1].y = None
    assert up(p, 1, 1, ads, 2, None) == 1003              # the up-projection needs somewhere to add to
    ads[1].y = p
    assert up(p, 0, 1, ads, 2, None) == 1001 and up(p, 257, 1, ads, 2, None) == 1001   # pieces of t per row


def test_base_launch_with_down_projection_validation(lib):
    keep, p = buf(1 << 16)
    probs = (_lib.Problem * 2)()
    for rec in probs:
        rec.x = rec.qweight = rec.y = p
        rec.M, rec.N, rec.K, rec.G, rec.prepacked = 2, 64, 256, 128, 1
    ads = (_lib.LoraAdapter * 2)()
    for ad in ads:
        ad.A, ad.B, ad.y, ad.N, ad.r, ad.scaling, ad.weights_fp32 = p, p, p, 64, 8, 2.0, 1
    f = lib.vrl_int4_gemv_prepacked_lora_bf16
    assert f(probs, 2, None, 2, p, None) == 1003 and f(probs, 2, ads, 2, None, None) == 1003
    assert f(probs, 2, ads, 2, p + 4, None) == 1002
    assert f(probs, 2, ads, 0, p, None) == 1001 and f(probs, 2, ads, 5, p, None) == 1001
    probs[1].x = p + 512
    assert f(probs, 2, ads, 2, p, None) == 1001          # every problem reads the adapters' input
    probs[1].x, probs[1].M = p, 1
    assert f(probs, 2, ads, 2, p, None) == 1001
    probs[1].M, probs[1].fused_gate_up = 2, 1
    assert f(probs, 2, ads, 2, p, None) == 1001          # no fused gate|up problem beside adapters
    probs[1].fused_gate_up = 0
    ads[1].r = 12
    assert f(probs, 2, ads, 2, p, None) == 1001


def test_base_launch_with_up_projection_validation(lib):
    keep, p = buf(1 << 16)
    prob = (_lib.Problem * 1)()
    prob[0].x = prob[0].qweight = prob[0].y = p
    prob[0].M, prob[0].N, prob[0].K, prob[0].G, prob[0].prepacked = 2, 64, 256, 128, 1
    ad = (_lib.LoraAdapter * 1)()
    ad[0].A, ad[0].B, ad[0].y, ad[0].N, ad[0].r, ad[0].scaling, ad[0].weights_fp32 = p, p, p, 64, 8, 2.0, 1
    f = lib.vrl_int4_gemv_prepacked_lora_up_bf16
    assert f(prob, None, p, 1, None) == 1003 and f(prob, ad, None, 1, None) == 1003 and f(None, ad, p, 1, None) == 1003
    assert f(prob, ad, p + 4, 1, None) == 1002
    assert f(prob, ad, p, 0, None) == 1001 and f(prob, ad, p, 257, None) == 1001
    ad[0].N = 32
    assert f(prob, ad, p, 1, None) == 1001               # the adapter's width is the problem's
    ad[0].N, ad[0].r = 64, 12
    assert f(prob, ad, p, 1, None) == 1001
    ad[0].r, ad[0].B = 8, None
    assert f(prob, ad, p, 1, None) == 1003
    ad[0].B, prob[0].fused_gate_up, prob[0].N = p, 1, 64
    assert f(prob, ad, p, 1, None) == 1001               # not beside a fused gate|up problem


def test_cfg_sample_validation(lib):
    keep, p = buf(4096)
    f = lib.vrl_cfg_sample_bf16
    assert f(None, p, p, p, 1, 16, 1.0, 1.0, None) == 1003
    assert f(p, p, p, None, 1, 16, 1.0, 1.0, None) == 1003
    assert f(p, p, p, p, 0, 16, 1.0, 1.0, None) == 1001
    assert f(p, p, p, p, 1, 0, 1.0, 1.0, None) == 1001
    assert f(p, p, p, p, 1, 16, 1.0, 0.0, None) == 1001          # temperature must be positive
    assert f(p, p, p, p, 1, 16, 1.0, float("nan"), None) == 1001
    assert f(p + 1, p, p, p, 1, 16, 1.0, 1.0, None) == 1002
    assert f(p, p, p + 4, p, 1, 16, 1.0, 1.0, None) == 1002      # int64 output


def test_epilogue_launch_validation(lib):
    keep, p = buf(1 << 16)
    prob = (_lib.Problem * 1)()
    prob[0].x = prob[0].qweight = prob[0].y = p
    prob[0].M, prob[0].N, prob[0].K, prob[0].G, prob[0].prepacked = 2, 64, 256, 128, 1
    epi = _lib.Epilogue()
    epi.bias, epi.activation = p, _lib.ACT_GELU
    f = lib.vrl_int4_gemv_prepacked_epilogue_bf16
    assert f(prob, None, None, None) == 1003 and f(None, None, ctypes.byref(epi), None) == 1003
    epi.activation = 7
    assert f(prob, None, ctypes.byref(epi), None) == 1001          # an activation the library does not know
    epi.activation, epi.bias = _lib.ACT_GELU, p + 1
    assert f(prob, None, ctypes.byref(epi), None) == 1002
    epi.bias, prob[0].fused_gate_up = p, 1
    assert f(prob, None, ctypes.byref(epi), None) == 1001          # a plain problem only
    prob[0].fused_gate_up, prob[0].prepacked = 0, 0
    assert f(prob, None, ctypes.byref(epi), None) == 1001


def test_head_sample_extras_validation(lib):
    keep, p = buf(1 << 20)
    p = (p + 255) & ~255
    head = _lib.Problem()
    head.x = head.qweight = p
    head.M, head.N, head.K, head.G, head.prepacked = 2, 64, 256, 128, 1
    need = lib.vrl_int4_head_sample_workspace_bytes(1, 64)
    assert need > 0 and need % 256 == 0
    f = lib.vrl_int4_head_sample_ex_bf16
    ex = _lib.HeadExtras()
    assert f(ctypes.byref(head), None, p, p, p, 1, 5.0, 1.0, p, need, None) == 1003
    ex.embed_table = p
    assert f(ctypes.byref(head), ctypes.byref(ex), p, p, p, 1, 5.0, 1.0, p, need, None) == 1003   # no destination
    ex.next_embeds, ex.embed_dim = p, 12
    assert f(ctypes.byref(head), ctypes.byref(ex), p, p, p, 1, 5.0, 1.0, p, need, None) == 1001   # 16-byte rows
    ex.embed_dim, ex.next_embeds = 16, p + 2
    assert f(ctypes.byref(head), ctypes.byref(ex), p, p, p, 1, 5.0, 1.0, p, need, None) == 1002
    ex.next_embeds, ex.tokens = p, p
    assert f(ctypes.byref(head), ctypes.byref(ex), p, p, p, 1, 5.0, 1.0, p, need, None) == 1003   # tokens need a position
    ex.position, ex.token_stride = p, 0
    assert f(ctypes.byref(head), ctypes.byref(ex), p, p, p, 1, 5.0, 1.0, p, need, None) == 1001
    ex.token_stride, ex.position = 8, p + 4
    assert f(ctypes.byref(head), ctypes.byref(ex), p, p, p, 1, 5.0, 1.0, p, need, None) == 1002
    ex.position = p
    assert f(ctypes.byref(head), ctypes.byref(ex), p, p, p, 1, 5.0, 1.0, p, need - 256, None) == 1001  # workspace too small


def test_step_call_records_hold_the_arguments_by_type_and_the_walk_reports_the_failing_call():
    """``vrl_decode_run_calls``: arguments go to the pointer / integer / float slots in declaration order; a NULL
    list, a negative count and an unknown kind are refused before anything is launched, the index of the call
    that failed is reported."""
    import ctypes

    lib = _lib.load()
    norm = _lib.Norm()
    table = _lib.step_calls([
        (lib.vrl_add_rmsnorm_bf16, (16, 32, 48, None, 80, 7, 2048, 0.5)),
        (lib.vrl_int4_gemv_prepacked_norm_bf16, ((_lib.Problem * 2)(), 2, ctypes.byref(norm))),
    ])
    assert table[0].kind == 6 and list(table[0].p[:5]) == [16, 32, 48, None, 80]
    assert list(table[0].i[:2]) == [7, 2048] and table[0].f[0] == 0.5
    assert table[1].kind == 2 and table[1].i[0] == 2 and table[1].p[1] == ctypes.addressof(norm)
    with pytest.raises(ValueError):
        _lib.step_calls([(lib.vrl_add_rmsnorm_bf16, (1, 2, 3))])
    failed = ctypes.c_int(-1)
    assert lib.vrl_decode_run_calls(None, 1, ctypes.byref(failed), None) == 1003
    assert lib.vrl_decode_run_calls(table, -1, ctypes.byref(failed), None) == 1001
    assert lib.vrl_decode_run_calls(table, 0, ctypes.byref(failed), None) == 0 and failed.value == -1
    bad = (_lib.StepCall * 2)()
    bad[0].kind, bad[1].kind = 6, 99      # a norm over NULL tensors, then an unknown entry point
    assert lib.vrl_decode_run_calls(bad, 2, ctypes.byref(failed), None) == 1003 and failed.value == 0
    bad[0].kind = 99
    assert lib.vrl_decode_run_calls(bad, 2, None, None) == 1001
