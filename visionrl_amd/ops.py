"""Torch operators over the HIP library (namespace ``vrl_hip``).

``vrl_hip::int4_gemv``          y[M,N]  = x[M,K] . dequant(W)^T
``vrl_hip::int4_dequant``       W[N,K]  bf16, bit-exact canonical tile
``vrl_hip::int4_gate_up_silu``  y[M,I]  = silu(x . Wg^T) * (x . Wu^T)

They stand where the reference calls bf16 ``nn.Linear`` modules during rollout
decode (``vrl/models/families/janus_pro/policy.py:673-678`` trunk,
``policy.py:138-160`` head).  Contract violations raise ``ValueError`` /
``TypeError`` before anything is enqueued, in the raise-on-violation style of the
reference's step functions (``policy.py:585-601``).  The operators run only on a
ROCm device through the HIP library: there is no CPU implementation, and a
missing library raises ``Int4LibraryError``.
"""

from __future__ import annotations

import contextlib
import ctypes

import torch

from . import _lib
from .int4_format import check_packed

__all__ = ["int4_gemv", "int4_dequant", "int4_gate_up_silu", "int4_gemv_into", "int4_prepack",
           "PrepackedWeight", "GroupedGemv", "DirectGemv", "int4_gemv_prepacked_into",
           "int4_gemv_prepacked_multi_into", "DirectCall", "cfg_sample", "head_sample", "head_sample_supported",
           "head_sample_workspace", "EpilogueGemv", "add_rmsnorm", "rope_attn_split_workspace",
           "rope_attn_decode", "LoraAdd"]


def _stream_handle(device: torch.device) -> int:
    return int(torch.cuda.current_stream(device).cuda_stream)


_NULL = contextlib.nullcontext()


def _on(device: torch.device):
    """Context that makes ``device`` current; free when it already is (the decode-loop case)."""
    if device.index is None or torch.cuda.current_device() == device.index:
        return _NULL
    return torch.cuda.device(device)


def _require_device(name: str, t: torch.Tensor, device: torch.device | None = None) -> torch.device:
    if t.device.type != "cuda":
        raise ValueError(
            f"{name} must live on a ROCm device (got {t.device}); the int4 operators have no CPU path")
    if device is not None and t.device != device:
        raise ValueError(f"{name} is on {t.device}, expected {device}")
    if not t.is_contiguous():
        raise ValueError(f"{name} must be contiguous")
    return t.device


def _check_call(x, qweight, scales, qzeros, group_size):
    if x.dtype != torch.bfloat16:
        raise TypeError(f"x must be bfloat16, got {x.dtype}")
    if x.dim() != 2:
        raise ValueError("x must be [M, K]")
    N, K, _ = check_packed(qweight, scales, qzeros, group_size)
    if x.shape[1] != K:
        raise ValueError(f"x has K={x.shape[1]}, packed weights have K={K}")
    if x.shape[0] < 1:
        raise ValueError("x needs at least one row")
    dev = _require_device("x", x)
    for name, t in (("qweight", qweight), ("scales", scales), ("qzeros", qzeros)):
        _require_device(name, t, dev)
    return x.shape[0], N, K, dev


@torch.library.custom_op("vrl_hip::int4_gemv", mutates_args=())
def int4_gemv(x: torch.Tensor, qweight: torch.Tensor, scales: torch.Tensor,
              qzeros: torch.Tensor, group_size: int) -> torch.Tensor:
    M, N, K, dev = _check_call(x, qweight, scales, qzeros, group_size)
    lib = _lib.load()
    y = torch.empty((M, N), dtype=torch.bfloat16, device=dev)
    with torch.cuda.device(dev):
        rc = lib.vrl_int4_gemv_bf16(x.data_ptr(), qweight.data_ptr(), scales.data_ptr(),
                                    qzeros.data_ptr(), y.data_ptr(), M, N, K, int(group_size),
                                    _stream_handle(dev))
    _lib.check(rc, "vrl_int4_gemv_bf16")
    return y


@int4_gemv.register_fake
def _(x, qweight, scales, qzeros, group_size):
    return x.new_empty((x.shape[0], qweight.shape[0]))


def int4_gemv_into(y: torch.Tensor, x: torch.Tensor, qweight: torch.Tensor, scales: torch.Tensor,
                   qzeros: torch.Tensor, group_size: int) -> torch.Tensor:
    """Lean eager form of ``int4_gemv``: writes into a caller-provided ``y[M,N]``.

    No allocation and no operator dispatch, for decode loops that call the same
    layer thousands of times; shapes and dtypes are still checked (by the
    library for the shape rules, here for the rest).
    """
    if x.dtype != torch.bfloat16 or y.dtype != torch.bfloat16 or scales.dtype != torch.bfloat16:
        raise TypeError("x, y and scales must be bfloat16")
    if qweight.dtype != torch.int32 or qzeros.dtype != torch.int32:
        raise TypeError("qweight and qzeros must be int32")
    if x.dim() != 2 or y.dim() != 2 or qweight.dim() != 2:
        raise ValueError("x, y and qweight must be 2-D")
    M, K = x.shape
    N = qweight.shape[0]
    if qweight.shape[1] * 8 != K or tuple(y.shape) != (M, N):
        raise ValueError(f"shape mismatch: x {tuple(x.shape)}, qweight {tuple(qweight.shape)}, y {tuple(y.shape)}")
    groups = K // int(group_size) if group_size else 0
    if tuple(scales.shape) != (N, groups) or tuple(qzeros.shape) != (N, (groups + 7) // 8):
        raise ValueError("scales / qzeros do not match qweight and group_size")
    dev = x.device
    for name, t in (("x", x), ("y", y), ("qweight", qweight), ("scales", scales), ("qzeros", qzeros)):
        if t.device != dev or dev.type != "cuda":
            raise ValueError(f"{name} must live on the same ROCm device; the int4 operators have no CPU path")
        if not t.is_contiguous():
            raise ValueError(f"{name} must be contiguous")
    rc = _lib.load().vrl_int4_gemv_bf16(x.data_ptr(), qweight.data_ptr(), scales.data_ptr(),
                                        qzeros.data_ptr(), y.data_ptr(), M, N, K, int(group_size),
                                        _stream_handle(dev))
    _lib.check(rc, "vrl_int4_gemv_bf16")
    return y


@torch.library.custom_op("vrl_hip::int4_dequant", mutates_args=())
def int4_dequant(qweight: torch.Tensor, scales: torch.Tensor, qzeros: torch.Tensor,
                 group_size: int) -> torch.Tensor:
    N, K, _ = check_packed(qweight, scales, qzeros, group_size)
    dev = _require_device("qweight", qweight)
    _require_device("scales", scales, dev)
    _require_device("qzeros", qzeros, dev)
    lib = _lib.load()
    w = torch.empty((N, K), dtype=torch.bfloat16, device=dev)
    with torch.cuda.device(dev):
        rc = lib.vrl_int4_dequant_bf16(qweight.data_ptr(), scales.data_ptr(), qzeros.data_ptr(),
                                       w.data_ptr(), N, K, int(group_size), _stream_handle(dev))
    _lib.check(rc, "vrl_int4_dequant_bf16")
    return w


@int4_dequant.register_fake
def _(qweight, scales, qzeros, group_size):
    return scales.new_empty((qweight.shape[0], qweight.shape[1] * 8))


@torch.library.custom_op("vrl_hip::int4_gate_up_silu", mutates_args=())
def int4_gate_up_silu(x: torch.Tensor, qweight_gu: torch.Tensor, scales_gu: torch.Tensor,
                      qzeros_gu: torch.Tensor, group_size: int) -> torch.Tensor:
    M, N2, K, dev = _check_call(x, qweight_gu, scales_gu, qzeros_gu, group_size)
    if N2 % 2 != 0:
        raise ValueError("gate||up operand needs an even number of rows")
    inter = N2 // 2
    lib = _lib.load()
    y = torch.empty((M, inter), dtype=torch.bfloat16, device=dev)
    with torch.cuda.device(dev):
        rc = lib.vrl_int4_gate_up_silu_bf16(x.data_ptr(), qweight_gu.data_ptr(), scales_gu.data_ptr(),
                                            qzeros_gu.data_ptr(), y.data_ptr(), M, inter, K,
                                            int(group_size), _stream_handle(dev))
    _lib.check(rc, "vrl_int4_gate_up_silu_bf16")
    return y


@int4_gate_up_silu.register_fake
def _(x, qweight_gu, scales_gu, qzeros_gu, group_size):
    return x.new_empty((x.shape[0], qweight_gu.shape[0] // 2))


class PrepackedWeight:
    """A weight repacked once for the grouped and plan-free launches (group sizes 32, 64, 128).

    ``blob`` is an opaque ``uint8`` device tensor made by the library from the
    canonical ``(qweight, scales, qzeros)`` triple; ``N``, ``K`` and
    ``group_size`` describe the operand it stands for.  The weights the kernels
    rebuild from it are bit for bit the canonical dequantised tile.
    """

    def __init__(self, blob: torch.Tensor, N: int, K: int, group_size: int):
        self.blob, self.N, self.K, self.group_size = blob, int(N), int(K), int(group_size)

    @staticmethod
    def supported(N: int, K: int, group_size: int) -> bool:
        return _lib.load().vrl_int4_prepacked_bytes(int(N), int(K), int(group_size)) > 0

    def direct_slab_rows(self, fused: bool = False) -> int:
        """Activation rows one record of a plan-free launch carries for this weight.

        A lower bound of the library's rule: the staged rows (K padded to 512, 8 elements
        of row padding) and the partial tiles of the K-split (at most 15 KiB, twice that for
        gate||up) fit 150 KiB of LDS, 16 rows at most.
        """
        nsc = (self.K + 511) // 512
        spare = 150 * 1024 - 15 * 1024 * (2 if fused else 1)
        return max(0, min(16, spare // ((nsc * 512 + 8) * 2)))

    def direct_rows(self, fused: bool = False, weights: int = 1) -> int:
        """Most activation rows a plan-free launch (:class:`DirectGemv`) takes for this weight
        when ``weights`` such problems share the launch: the library cuts the rows into slabs
        and a launch holds at most eight of them.  Capped at 32 rows: beyond that every slab
        streams the weight again and a plan (:class:`GroupedGemv`) is the better launch."""
        slab = self.direct_slab_rows(fused)
        return min(32, slab * (DirectGemv.MAX_RECORDS // max(1, int(weights))))


def int4_prepack(qweight: torch.Tensor, scales: torch.Tensor, qzeros: torch.Tensor,
                 group_size: int) -> PrepackedWeight:
    """Repack a canonical operand triple on its device; raises ``ValueError`` if the
    shape has no prepacked form (group size other than 128)."""
    N, K, _ = check_packed(qweight, scales, qzeros, group_size)
    dev = _require_device("qweight", qweight)
    _require_device("scales", scales, dev)
    _require_device("qzeros", qzeros, dev)
    lib = _lib.load()
    nbytes = lib.vrl_int4_prepacked_bytes(N, K, int(group_size))
    if nbytes == 0:
        raise ValueError(f"no prepacked form for N={N}, K={K}, group_size={group_size} "
                         "(needs group_size 128)")
    blob = torch.empty(nbytes, dtype=torch.uint8, device=dev)
    with torch.cuda.device(dev):
        rc = lib.vrl_int4_prepack(qweight.data_ptr(), scales.data_ptr(), qzeros.data_ptr(),
                                  blob.data_ptr(), N, K, int(group_size), _stream_handle(dev))
    _lib.check(rc, "vrl_int4_prepack")
    return PrepackedWeight(blob, N, K, group_size)


class GroupedGemv:
    """Several independent int4 GEMVs enqueued as one kernel launch.

    ``problems`` is a list of ``(x, qweight, scales, qzeros, group_size, fused)``
    tuples, or ``(x, prepacked_weight, fused)`` with a :class:`PrepackedWeight`;
    outputs are allocated once here and overwritten by every :meth:`launch`.  The
    plan (pointer table) is validated and built on the host by the library,
    copied to the device once, and stays valid while the tensors captured here
    are alive and not reallocated.
    """

    MAX_ROWS = 16            # activation rows one canonical record of the plan may carry
    MAX_ROWS_PREPACKED = 32  # ... and one prepacked record (two MFMA row blocks per weight tile)

    def __init__(self, problems):
        if not problems:
            raise ValueError("GroupedGemv needs at least one problem")
        lib = _lib.load()
        self._keep = []
        self.outputs = []
        dev = None
        records = []
        for prob in problems:
            if len(prob) == 3:
                x, pw, fused = prob
                if not isinstance(pw, PrepackedWeight):
                    raise TypeError("(x, weight, fused) problems take a PrepackedWeight")
                if x.dtype != torch.bfloat16 or x.dim() != 2 or x.shape[1] != pw.K or x.shape[0] < 1:
                    raise ValueError(f"x must be bfloat16 [M, {pw.K}]")
                d = _require_device("x", x)
                _require_device("prepacked blob", pw.blob, d)
                M, N, K, group_size = x.shape[0], pw.N, pw.K, pw.group_size
                ptrs = (pw.blob.data_ptr(), 0, 0)
                keep = (x, pw)
                prepacked = 1
            else:
                x, qweight, scales, qzeros, group_size, fused = prob
                M, N, K, d = _check_call(x, qweight, scales, qzeros, group_size)
                ptrs = (qweight.data_ptr(), scales.data_ptr(), qzeros.data_ptr())
                keep = (x, qweight, scales, qzeros)
                prepacked = 0
            if dev is None:
                dev = d
            elif d != dev:
                raise ValueError("all problems of a grouped launch must share one device")
            if fused and N % 2 != 0:
                raise ValueError("gate||up operand needs an even number of rows")
            y = torch.empty((M, N // 2 if fused else N), dtype=torch.bfloat16, device=dev)
            self._keep.append(keep)
            self.outputs.append(y)
            # one record per slab of activation rows (row slices stay contiguous)
            rows = self.MAX_ROWS_PREPACKED if prepacked else self.MAX_ROWS
            for m0 in range(0, M, rows):
                m1 = min(M, m0 + rows)
                records.append((x[m0:m1].data_ptr(), *ptrs, y[m0:m1].data_ptr(), m1 - m0, N, K,
                                int(group_size), 1 if fused else 0, prepacked))
        n = len(records)
        table = (_lib.Problem * n)()
        for rec, vals in zip(table, records):
            (rec.x, rec.qweight, rec.scales, rec.qzeros, rec.y,
             rec.M, rec.N, rec.K, rec.G, rec.fused_gate_up, rec.prepacked) = vals
        size = lib.vrl_int4_grouped_plan_size(n)
        host = torch.empty(size, dtype=torch.uint8)
        self.info = _lib.PlanInfo()
        with torch.cuda.device(dev):  # the plan is sized for this device's CU count
            rc = lib.vrl_int4_grouped_plan_build(table, n, host.data_ptr(), size,
                                                 ctypes.byref(self.info))
        _lib.check(rc, "vrl_int4_grouped_plan_build")
        self.device = dev
        self.plan = host.to(dev)

    def launch(self):
        lib = _lib.load()
        with _on(self.device):
            rc = lib.vrl_int4_gemv_grouped_bf16(self.plan.data_ptr(), ctypes.byref(self.info),
                                                _stream_handle(self.device))
        _lib.check(rc, "vrl_int4_gemv_grouped_bf16")
        return self.outputs


class DirectGemv:
    """One to eight prepacked GEMVs launched together without a plan in device memory.

    The decode-time form of a linear (or of the q|k|v / gate|up linears of one decoder
    layer, ``vrl/models/families/janus_pro/policy.py:673-678``): the problem records
    travel as kernel arguments, so a launch is one memory round trip.  ``problems`` is a
    list of ``(x, prepacked_weight, fused)``; every x has at most 32 rows, which the library
    takes in slabs of up to 16 (fewer for long K), eight slabs per launch at most.  Outputs
    are allocated here once and overwritten by every :meth:`launch`; the record table is
    built once, the tensors captured here must stay alive and in place.
    """

    MAX_PROBLEMS = 8
    MAX_ROWS = 32
    MAX_RECORDS = 8   # row slabs of all problems of one launch

    def __init__(self, problems, outputs=None, norm=None):
        if not 1 <= len(problems) <= self.MAX_PROBLEMS:
            raise ValueError(f"DirectGemv takes 1 to {self.MAX_PROBLEMS} problems")
        self.norm = None
        self._keep = []
        self.outputs = []
        self.table = (_lib.Problem * len(problems))()
        dev = None
        for i, (rec, (x, pw, fused)) in enumerate(zip(self.table, problems)):
            if not isinstance(pw, PrepackedWeight):
                raise TypeError("DirectGemv problems take a PrepackedWeight")
            if x.dtype != torch.bfloat16 or x.dim() != 2 or x.shape[1] != pw.K or not 1 <= x.shape[0] <= self.MAX_ROWS:
                raise ValueError(f"x must be bfloat16 [1..{self.MAX_ROWS}, {pw.K}]")
            if not x.is_contiguous():
                raise ValueError("x must be contiguous")
            d = _require_device("x", x)
            _require_device("prepacked blob", pw.blob, d)
            if dev is None:
                dev = d
            elif d != dev:
                raise ValueError("all problems of one launch must share one device")
            if fused and pw.N % 2 != 0:
                raise ValueError("gate||up operand needs an even number of rows")
            cols = pw.N // 2 if fused else pw.N
            if outputs is None:
                y = torch.empty((x.shape[0], cols), dtype=torch.bfloat16, device=dev)
            else:
                y = outputs[i]
                if y.dtype != torch.bfloat16 or tuple(y.shape) != (x.shape[0], cols) or not y.is_contiguous():
                    raise ValueError(f"output {i} must be contiguous bfloat16 [{x.shape[0]}, {cols}]")
                _require_device("y", y, dev)
            self._keep.append((x, pw))
            self.outputs.append(y)
            rec.x, rec.qweight, rec.scales, rec.qzeros, rec.y = x.data_ptr(), pw.blob.data_ptr(), 0, 0, y.data_ptr()
            rec.M, rec.N, rec.K, rec.G = x.shape[0], pw.N, pw.K, pw.group_size
            rec.fused_gate_up, rec.prepacked = (1 if fused else 0), 1
        self.device = dev
        if norm is not None:
            self._set_norm(problems, *norm)

    def _set_norm(self, problems, residual, weight, eps, h_out):
        """``norm=(residual | None, weight, eps, h_out | None)``: every problem then multiplies
        ``weight * rmsnorm(x + residual)`` instead of its ``x`` (the same tensor for all of them), the
        add and norm of ``LlamaDecoderLayer.forward`` in front of q|k|v or gate|up; ``h_out``
        receives ``x + residual`` and must be a buffer of its own."""
        x = problems[0][0]
        if any(prob[0] is not x for prob in problems):
            raise ValueError("a normalised launch takes one input tensor for all its problems")
        if weight.dtype != torch.bfloat16 or tuple(weight.shape) != (x.shape[1],) or not weight.is_contiguous():
            raise ValueError(f"norm weight must be contiguous bfloat16 [{x.shape[1]}]")
        _require_device("norm weight", weight, self.device)
        for name, t in (("residual", residual), ("h_out", h_out)):
            if t is not None:
                if t.dtype != torch.bfloat16 or t.shape != x.shape or not t.is_contiguous():
                    raise ValueError(f"{name} must be contiguous bfloat16 {tuple(x.shape)}")
                _require_device(name, t, self.device)
        rec = _lib.Norm()
        rec.x, rec.weight, rec.eps = x.data_ptr(), weight.data_ptr(), float(eps)
        rec.residual = residual.data_ptr() if residual is not None else None
        rec.h_out = h_out.data_ptr() if h_out is not None else None
        self.norm = rec
        self._keep.append((residual, weight, h_out))

    def launch(self, lora_down: "LoraAdd | None" = None, lora_up: "LoraAdd | None" = None):
        """``lora_down``: a :class:`LoraAdd` over the input every problem of this launch reads; its
        down-projection then runs in the same launch (in place of its ``launch_down``).
        ``lora_up``: a :class:`LoraAdd` with one adapter over this launch's one output, whose ``t`` is
        ready; the launch adds its up-projection before it stores (in place of its ``launch_up``)."""
        lib = _lib.load()
        with _on(self.device):
            if lora_up is not None:
                if lora_down is not None or self.norm is not None or len(self.table) != 1 or \
                        len(lora_up.table) != 1 or lora_up.table[0].y != self.table[0].y:
                    raise ValueError("an up-projection joins the launch of the one problem whose output it adds to")
                rc = lib.vrl_int4_gemv_prepacked_lora_up_bf16(self.table, lora_up.table, lora_up.t.data_ptr(),
                                                              lora_up.parts, _stream_handle(self.device))
            elif lora_down is not None:
                if lora_down.parts != 1:
                    raise ValueError("the adapters' down-projection joins the launch in one piece")
                if self.norm is not None:   # base projections and adapters over the normalised rows (K <= 2048)
                    rc = lib.vrl_int4_gemv_prepacked_norm_lora_bf16(
                        self.table, len(self.table), ctypes.byref(self.norm), lora_down.table, len(lora_down.table),
                        lora_down.t.data_ptr(), _stream_handle(self.device))
                else:
                    rc = lib.vrl_int4_gemv_prepacked_lora_bf16(self.table, len(self.table), lora_down.table,
                                                               len(lora_down.table), lora_down.t.data_ptr(),
                                                               _stream_handle(self.device))
            elif self.norm is not None:
                rc = lib.vrl_int4_gemv_prepacked_norm_bf16(self.table, len(self.table), ctypes.byref(self.norm),
                                                           _stream_handle(self.device))
            else:
                rc = lib.vrl_int4_gemv_prepacked_bf16(self.table, len(self.table), _stream_handle(self.device))
        _lib.check(rc, "vrl_int4_gemv_prepacked_bf16")
        return self.outputs


def int4_gemv_prepacked_into(y: torch.Tensor, x: torch.Tensor, weight: PrepackedWeight,
                             fused: bool = False) -> torch.Tensor:
    """``y = x . dequant(weight)^T`` over a prepacked weight, one plan-free launch.

    Lean eager path (module forward): bf16 contiguous ``x [M <= weight.direct_rows(), K]``
    and ``y`` on the weight's device; shape preconditions are checked by the library.
    """
    if x.dtype != torch.bfloat16 or y.dtype != torch.bfloat16 or not x.is_contiguous() or not y.is_contiguous():
        raise ValueError("x and y must be contiguous bfloat16")
    if x.dim() != 2 or x.shape[1] != weight.K or tuple(y.shape) != (x.shape[0], weight.N // 2 if fused else weight.N):
        raise ValueError("x must be [M, K] and y [M, N] for this weight")
    dev = _require_device("x", x)
    _require_device("y", y, dev)
    _require_device("prepacked blob", weight.blob, dev)
    rec = _lib.Problem()
    rec.x, rec.qweight, rec.y = x.data_ptr(), weight.blob.data_ptr(), y.data_ptr()
    rec.M, rec.N, rec.K, rec.G = x.shape[0], weight.N, weight.K, weight.group_size
    rec.fused_gate_up, rec.prepacked = (1 if fused else 0), 1
    with _on(dev):
        rc = _lib.load().vrl_int4_gemv_prepacked_bf16(ctypes.byref(rec), 1, _stream_handle(dev))
    _lib.check(rc, "vrl_int4_gemv_prepacked_bf16")
    return y


def int4_gemv_prepacked_multi_into(ys, x: torch.Tensor, weights) -> None:
    """One plan-free launch for up to eight prepacked weights applied to the same ``x`` (q|k|v).

    Lean eager path like :func:`int4_gemv_prepacked_into`: ``x`` bf16 contiguous ``[M, K]``,
    ``ys[i]`` bf16 contiguous ``[M, weights[i].N]``, all on one device.
    """
    n = len(weights)
    if not 1 <= n <= DirectGemv.MAX_PROBLEMS or len(ys) != n:
        raise ValueError(f"1 to {DirectGemv.MAX_PROBLEMS} weights, one output each")
    if x.dtype != torch.bfloat16 or x.dim() != 2 or not x.is_contiguous():
        raise ValueError("x must be contiguous bfloat16 [M, K]")
    dev = _require_device("x", x)
    table = (_lib.Problem * n)()
    for rec, w, y in zip(table, weights, ys):
        if w.K != x.shape[1] or y.dtype != torch.bfloat16 or tuple(y.shape) != (x.shape[0], w.N) or \
                not y.is_contiguous():
            raise ValueError("every weight must take x's K and every output be contiguous bfloat16 [M, N]")
        _require_device("y", y, dev)
        _require_device("prepacked blob", w.blob, dev)
        rec.x, rec.qweight, rec.y = x.data_ptr(), w.blob.data_ptr(), y.data_ptr()
        rec.M, rec.N, rec.K, rec.G, rec.prepacked = x.shape[0], w.N, w.K, w.group_size, 1
    with _on(dev):
        rc = _lib.load().vrl_int4_gemv_prepacked_bf16(table, n, _stream_handle(dev))
    _lib.check(rc, "vrl_int4_gemv_prepacked_bf16")


class EpilogueGemv:
    """One prepacked linear with its bias and a following GELU applied before the store, one plan-free launch:
    ``y = act(bf16(bf16(x . W^T) + bias))``, optionally over ``weight * rmsnorm(x + residual)`` instead of ``x``.

    The first half of Janus' two-layer image-token head (``Linear``, ``GELU``, ``Linear``; called through
    ``gen_head`` at ``vrl/models/families/janus_pro/policy.py:138-160``) and any biased linear.  ``x`` is a
    contiguous bf16 ``[M <= 32, K]`` tensor; ``bias`` bf16 ``[N]`` or ``None``; ``gelu`` the exact (erf) form of
    ``torch.nn.GELU()``; ``norm = (residual | None, weight, eps)`` as in :class:`DirectGemv` (K <= 4096);
    ``residual`` (bf16 ``[M, N]``) is added last, ``y = bf16(residual + ...)``: the residual stream that the
    outputs of ``o_proj`` and ``down_proj`` join in a decoder layer.  The record is built once; the tensors
    captured here must stay alive and in place.
    """

    def __init__(self, x: torch.Tensor, weight: "PrepackedWeight", bias: torch.Tensor | None = None,
                 gelu: bool = False, norm=None, out: torch.Tensor | None = None,
                 residual: torch.Tensor | None = None):
        self._gemv = DirectGemv([(x, weight, False)], outputs=None if out is None else [out],
                                norm=None if norm is None else (*norm, None))
        self.device = self._gemv.device
        if bias is not None:
            if bias.dtype != torch.bfloat16 or tuple(bias.shape) != (weight.N,) or not bias.is_contiguous():
                raise ValueError(f"bias must be contiguous bfloat16 [{weight.N}]")
            _require_device("bias", bias, self.device)
        self.output = self._gemv.outputs[0]
        if residual is not None:
            if residual.dtype != torch.bfloat16 or residual.shape != self.output.shape or not residual.is_contiguous():
                raise ValueError(f"residual must be contiguous bfloat16 {tuple(self.output.shape)}")
            _require_device("residual", residual, self.device)
        self.epilogue = _lib.Epilogue()
        self.epilogue.bias = bias.data_ptr() if bias is not None else None
        self.epilogue.residual = residual.data_ptr() if residual is not None else None
        self.epilogue.activation = _lib.ACT_GELU if gelu else _lib.ACT_NONE
        self._keep = (bias, residual)

    def launch(self) -> torch.Tensor:
        g = self._gemv
        with _on(self.device):
            rc = _lib.load().vrl_int4_gemv_prepacked_epilogue_bf16(
                g.table, ctypes.byref(g.norm) if g.norm is not None else None, ctypes.byref(self.epilogue),
                _stream_handle(self.device))
        _lib.check(rc, "vrl_int4_gemv_prepacked_epilogue_bf16")
        return self.output


def cfg_sample(logits: torch.Tensor, cfg_weight: float, temperature: float, *,
               generator: torch.Generator | None = None, noise: torch.Tensor | None = None):
    """CFG combine, softmax, one multinomial draw and its log-probability, in one launch.

    Stands for ``vrl/models/families/janus_pro/policy.py:686-693``: ``logits`` is the head's
    bf16 ``[2B, V]`` output with the conditional rows first; returns ``(sampled int64 [B],
    logprob float32 [B])``.  The draw consumes the random stream exactly as
    ``torch.multinomial(probs, 1)`` does (one ``exponential_(1)`` over a bf16 ``[B, V]``
    tensor), so a seeded rollout samples the same tokens; pass ``noise`` to supply the
    exponential draws yourself.
    """
    if logits.dtype != torch.bfloat16 or logits.dim() != 2 or logits.shape[0] % 2 != 0 or logits.shape[0] < 2:
        raise ValueError("logits must be bfloat16 [2B, V]: conditional rows, then unconditional rows")
    if not temperature > 0:
        raise ValueError("temperature must be positive")
    dev = _require_device("logits", logits)
    B, V = logits.shape[0] // 2, logits.shape[1]
    if noise is None:
        noise = torch.empty((B, V), dtype=torch.bfloat16, device=dev).exponential_(1.0, generator=generator)
    elif noise.dtype != torch.bfloat16 or tuple(noise.shape) != (B, V):
        raise ValueError(f"noise must be bfloat16 [{B}, {V}]")
    _require_device("noise", noise, dev)
    sampled = torch.empty(B, dtype=torch.int64, device=dev)
    logprob = torch.empty(B, dtype=torch.float32, device=dev)
    with _on(dev):
        rc = _lib.load().vrl_cfg_sample_bf16(logits.data_ptr(), noise.data_ptr(), sampled.data_ptr(),
                                             logprob.data_ptr(), B, V, float(cfg_weight), float(temperature),
                                             _stream_handle(dev))
    _lib.check(rc, "vrl_cfg_sample_bf16")
    return sampled, logprob


def head_sample_supported(rows: int, head: PrepackedWeight) -> bool:
    """Whether :func:`head_sample` takes ``rows = 2B`` activation rows for this head: the library's own
    rule (B <= 16, V a multiple of 16 up to 65536, the rows fit a workgroup's LDS beside the partial tiles)."""
    if rows < 2 or rows % 2 or rows > 32 or head.N < 16 or head.N > 65536 or head.N % 16:
        return False
    nsc = (head.K + 511) // 512
    if nsc > 16:
        return False
    ks = 16 if nsc > 8 else (8 if nsc > 4 else 4)
    tw = 16 // ks if rows >= 8 else 1
    lds = rows * (nsc * 512 + 8) * 2 + tw * (ks - 1) * (2 if rows > 16 else 1) * 64 * 16
    return lds <= 160 * 1024 - 64


def head_sample_workspace(B: int, V: int, device) -> torch.Tensor:
    """A workspace for :func:`head_sample` at batch ``B`` and vocabulary ``V`` (reusable by calls that
    do not overlap in time)."""
    nbytes = _lib.load().vrl_int4_head_sample_workspace_bytes(int(B), int(V))
    if nbytes == 0:
        raise ValueError(f"head_sample takes 1 <= B <= 16 and V a multiple of 16 up to 65536, got B={B}, V={V}")
    return torch.empty(nbytes, dtype=torch.uint8, device=device)


def head_sample(x: torch.Tensor, head: PrepackedWeight, cfg_weight: float, temperature: float, *,
                generator: torch.Generator | None = None, noise: torch.Tensor | None = None,
                logits_out: torch.Tensor | None = None, workspace: "torch.Tensor | str | None" = None, out=None,
                bias: torch.Tensor | None = None, bookkeeping=None, embedding=None, per_row: bool = False,
                active: torch.Tensor | None = None):
    """The image-token head and the sampling tail of a decode step in one launch.

    Stands for ``vrl/models/families/janus_pro/policy.py:684-693``: ``x`` is the bf16 ``[2B, K]``
    last hidden state (conditional rows first), ``head`` the prepacked ``gen_head`` weight
    ``[V, K]``; returns ``(sampled int64 [B], logprob float32 [B])`` like :func:`cfg_sample` over the
    head's logits, which are written to ``logits_out`` (bf16 ``[2B, V]``) only if that is given.
    The draw consumes the random stream as ``torch.multinomial(probs, 1)`` does; ``workspace`` is a
    tensor from :func:`head_sample_workspace` (made per call if omitted: pass one in a decode loop), or
    the string ``"static"`` for the library's own fixed scratch (``vrl_int4_head_sample_static_bf16``:
    B <= 16, V <= 16384, one call at a time per GPU); with ``noise`` and ``out = (sampled, logprob)``
    given as well, the call then allocates nothing.

    The parts of the step around it, done by the same call when given (``vrl_int4_head_sample_ex_bf16``):
    ``bias`` (bf16 ``[V]``) of a biased head, added to the rounded logits as the module adds it;
    ``bookkeeping = (tokens int64 [B, L], logprobs float32 [B, L], position int64 [1], slot int64 [1] | None)``:
    the draw and its log-probability are written at column ``position`` of the two buffers, ``position`` and
    ``slot`` are incremented (``policy.py:695-696`` over a device-side position); ``embedding = (table bf16
    [V, H], next bf16 [2B, H])``: rows ``b`` and ``B + b`` of ``next`` receive ``table[sampled[b]]``, the next
    input embedding of both rows of the pair (``policy.py:698-700`` with ``prepare_gen_img_embeds`` tabulated).
    ``per_row``: ``position`` is int64 ``[B]`` and ``slot`` int64 ``[2B]``, one counter per row, for rows that
    advance at different times; ``active`` (uint8 ``[B]``) then names the rows of this step's batch, the only
    ones written, counted on and given a next input.
    Raises ``ValueError`` for shapes the launch does not take (:func:`head_sample_supported`).
    """
    if x.dtype != torch.bfloat16 or x.dim() != 2 or x.shape[0] % 2 != 0 or x.shape[0] < 2 or x.shape[1] != head.K:
        raise ValueError(f"x must be bfloat16 [2B, {head.K}]: conditional rows, then unconditional rows")
    if not temperature > 0:
        raise ValueError("temperature must be positive")
    dev = _require_device("x", x)
    _require_device("prepacked blob", head.blob, dev)
    B, V = x.shape[0] // 2, head.N
    if not head_sample_supported(x.shape[0], head):
        raise ValueError(f"head_sample does not take {x.shape[0]} rows of K={head.K} for a head of {V} entries")
    if noise is None:
        noise = torch.empty((B, V), dtype=torch.bfloat16, device=dev).exponential_(1.0, generator=generator)
    elif noise.dtype != torch.bfloat16 or tuple(noise.shape) != (B, V):
        raise ValueError(f"noise must be bfloat16 [{B}, {V}]")
    _require_device("noise", noise, dev)
    if logits_out is not None:
        if logits_out.dtype != torch.bfloat16 or tuple(logits_out.shape) != (2 * B, V):
            raise ValueError(f"logits_out must be bfloat16 [{2 * B}, {V}]")
        _require_device("logits_out", logits_out, dev)
    static = isinstance(workspace, str) and workspace == "static"
    if workspace is None:
        workspace = head_sample_workspace(B, V, dev)
    elif not static and (workspace.dtype != torch.uint8 or workspace.device != dev or not workspace.is_contiguous()):
        raise ValueError("workspace must be a contiguous uint8 tensor on the device of x")
    if out is None:
        out = (torch.empty(B, dtype=torch.int64, device=dev), torch.empty(B, dtype=torch.float32, device=dev))
    sampled, logprob = out
    if sampled.dtype != torch.int64 or logprob.dtype != torch.float32 or tuple(sampled.shape) != (B,) or \
            tuple(logprob.shape) != (B,):
        raise ValueError(f"out must be (int64 [{B}], float32 [{B}])")
    _require_device("sampled", sampled, dev)
    _require_device("logprob", logprob, dev)
    rec = _lib.Problem()
    rec.x, rec.qweight, rec.y = x.data_ptr(), head.blob.data_ptr(), (logits_out.data_ptr() if logits_out is not None else None)
    rec.M, rec.N, rec.K, rec.G, rec.prepacked = 2 * B, V, head.K, head.group_size, 1
    extras = None
    if bias is not None or bookkeeping is not None or embedding is not None:
        if static:
            raise ValueError("the library's fixed scratch serves the plain call only")
        extras = _lib.HeadExtras()
        if bias is not None:
            if bias.dtype != torch.bfloat16 or tuple(bias.shape) != (V,) or not bias.is_contiguous():
                raise ValueError(f"bias must be contiguous bfloat16 [{V}]")
            _require_device("bias", bias, dev)
            extras.bias = bias.data_ptr()
        if bookkeeping is not None:
            tokens, logprobs, position, slot = bookkeeping
            if tokens.dtype != torch.int64 or logprobs.dtype != torch.float32 or tokens.dim() != 2 or \
                    tokens.shape != logprobs.shape or tokens.shape[0] != B or not tokens.is_contiguous() or \
                    not logprobs.is_contiguous():
                raise ValueError(f"bookkeeping buffers must be contiguous int64 / float32 [{B}, L]")
            for name, t, n in (("position", position, B if per_row else 1), ("slot", slot, 2 * B if per_row else 1)):
                if t is not None and (t.dtype != torch.int64 or t.numel() != n or not t.is_contiguous()):
                    raise ValueError(f"{name} must be a contiguous int64 device tensor of {n} element(s)")
            if active is not None:
                if not per_row or active.dtype != torch.uint8 or active.numel() != B or not active.is_contiguous():
                    raise ValueError(f"active goes with per_row and is a contiguous uint8 [{B}] tensor")
                _require_device("active", active, dev)
                extras.active = active.data_ptr()
            extras.position_per_row = 1 if per_row else 0
            for name, t in (("tokens", tokens), ("logprobs", logprobs), ("position", position), ("slot", slot)):
                if t is not None:
                    _require_device(name, t, dev)
            extras.tokens, extras.logprobs, extras.position = tokens.data_ptr(), logprobs.data_ptr(), position.data_ptr()
            extras.slot = slot.data_ptr() if slot is not None else None
            extras.token_stride = tokens.shape[1]
        if embedding is not None:
            table, nxt = embedding
            H = table.shape[-1]
            if table.dtype != torch.bfloat16 or tuple(table.shape) != (V, H) or not table.is_contiguous() or H % 8:
                raise ValueError(f"embedding table must be contiguous bfloat16 [{V}, H], H a multiple of 8")
            if nxt.dtype != torch.bfloat16 or nxt.numel() != 2 * B * H or not nxt.is_contiguous():
                raise ValueError(f"next embeddings must be contiguous bfloat16 with {2 * B} rows of {H}")
            _require_device("embedding table", table, dev)
            _require_device("next embeddings", nxt, dev)
            extras.embed_table, extras.next_embeds, extras.embed_dim = table.data_ptr(), nxt.data_ptr(), H
    with _on(dev):
        if extras is not None:
            rc = _lib.load().vrl_int4_head_sample_ex_bf16(ctypes.byref(rec), ctypes.byref(extras), noise.data_ptr(),
                                                          sampled.data_ptr(), logprob.data_ptr(), B, float(cfg_weight),
                                                          float(temperature), workspace.data_ptr(), workspace.numel(),
                                                          _stream_handle(dev))
        elif static:   # the library's own scratch: the call allocates nothing
            rc = _lib.load().vrl_int4_head_sample_static_bf16(ctypes.byref(rec), noise.data_ptr(), sampled.data_ptr(),
                                                              logprob.data_ptr(), B, float(cfg_weight),
                                                              float(temperature), _stream_handle(dev))
        else:
            rc = _lib.load().vrl_int4_head_sample_bf16(ctypes.byref(rec), noise.data_ptr(), sampled.data_ptr(),
                                                       logprob.data_ptr(), B, float(cfg_weight), float(temperature),
                                                       workspace.data_ptr(), workspace.numel(), _stream_handle(dev))
    _lib.check(rc, "vrl_int4_head_sample_bf16")
    return sampled, logprob


class DirectCall:
    """Reusable plan-free launch for one module's weight, or a q|k|v group: the eager decode path.

    Everything that does not change between calls (blob pointers, shapes) sits in a record
    table built once; a call fills in the activation pointer, the row count and the output
    pointers, allocates all outputs as one buffer, and launches.  The Python side of a decode
    step is host-bound, so this path validates only what can change (the caller, a module,
    owns the rest): ``x2d`` must be a contiguous bf16 ``[M, K]`` tensor on the weights' device.
    """

    def __init__(self, weights, fused: bool = False):
        if not 1 <= len(weights) <= DirectGemv.MAX_PROBLEMS:
            raise ValueError(f"1 to {DirectGemv.MAX_PROBLEMS} weights")
        self.table = (_lib.Problem * len(weights))()
        self.cols = []
        self.device = weights[0].blob.device
        self.K = weights[0].K
        for rec, w in zip(self.table, weights):
            if w.K != self.K or w.blob.device != self.device:
                raise ValueError("grouped weights take the same input on one device")
            rec.qweight, rec.N, rec.K, rec.G = w.blob.data_ptr(), w.N, w.K, w.group_size
            rec.fused_gate_up, rec.prepacked = (1 if fused else 0), 1
            self.cols.append(w.N // 2 if fused else w.N)
        self._keep = list(weights)
        self.max_rows = min(w.direct_rows(fused, len(weights)) for w in weights)
        self._fn = _lib.load().vrl_int4_gemv_prepacked_bf16
        self._n = len(weights)

    def __call__(self, x2d: torch.Tensor):
        M = x2d.shape[0]
        if self._n == 1:
            y = torch.empty((M, self.cols[0]), dtype=torch.bfloat16, device=x2d.device)
            rec = self.table[0]
            rec.x, rec.y, rec.M = x2d.data_ptr(), y.data_ptr(), M
            with _on(self.device):
                rc = self._fn(self.table, 1, torch.cuda.current_stream(self.device).cuda_stream)
            if rc:
                _lib.check(rc, "vrl_int4_gemv_prepacked_bf16")
            return [y]
        # every output starts on a 16-byte boundary of the one buffer
        sizes = [(M * c + 7) & ~7 for c in self.cols]
        buf = torch.empty(sum(sizes), dtype=torch.bfloat16, device=x2d.device)
        xp, base, off, outs = x2d.data_ptr(), buf.data_ptr(), 0, []
        for rec, c, size in zip(self.table, self.cols, sizes):
            rec.x, rec.y, rec.M = xp, base + 2 * off, M
            outs.append(buf[off:off + M * c].view(M, c))
            off += size
        with _on(self.device):
            rc = self._fn(self.table, self._n, torch.cuda.current_stream(self.device).cuda_stream)
        if rc:
            _lib.check(rc, "vrl_int4_gemv_prepacked_bf16")
        return outs


# ---------------------------------------------------------------------- decode-step kernels around the linears
def add_rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float, residual: torch.Tensor | None = None,
                *, h_out: torch.Tensor | None = None, y: torch.Tensor | None = None):
    """``LlamaRMSNorm`` of ``h = x (+ residual)`` over bf16 rows ``[M, K]``: returns ``(h, normed)``.

    The residual add of ``LlamaDecoderLayer.forward`` and the norm that follows it, in one launch
    (reached from ``vrl/models/families/janus_pro/policy.py:673-678``).  ``h_out`` / ``y`` may be
    given to reuse buffers; without a residual ``h`` is ``x`` itself.
    """
    if x.dtype != torch.bfloat16 or x.dim() != 2 or not x.is_contiguous():
        raise ValueError("x must be contiguous bfloat16 [M, K]")
    dev = _require_device("x", x)
    M, K = x.shape
    if weight.dtype != torch.bfloat16 or tuple(weight.shape) != (K,) or not weight.is_contiguous():
        raise ValueError(f"weight must be contiguous bfloat16 [{K}]")
    _require_device("weight", weight, dev)
    for name, t in (("residual", residual), ("h_out", h_out), ("y", y)):
        if t is not None:
            if t.dtype != torch.bfloat16 or tuple(t.shape) != (M, K) or not t.is_contiguous():
                raise ValueError(f"{name} must be contiguous bfloat16 [{M}, {K}]")
            _require_device(name, t, dev)
    if y is None:
        y = torch.empty_like(x)
    if residual is not None and h_out is None:
        h_out = torch.empty_like(x)
    with _on(dev):
        rc = _lib.load().vrl_add_rmsnorm_bf16(
            x.data_ptr(), residual.data_ptr() if residual is not None else None, weight.data_ptr(),
            h_out.data_ptr() if h_out is not None else None, y.data_ptr(), M, K, float(eps), _stream_handle(dev))
    _lib.check(rc, "vrl_add_rmsnorm_bf16")
    return (h_out if h_out is not None else x), y


def rope_attn_decode(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, k_cache: torch.Tensor,
                     v_cache: torch.Tensor, cos: torch.Tensor, sin: torch.Tensor, mask: torch.Tensor,
                     position: torch.Tensor, scaling: float, *, out: torch.Tensor | None = None,
                     lora: "LoraAdd | None" = None, out_lora: "LoraAdd | None" = None,
                     split_workspace: torch.Tensor | None = None, per_row: bool = False) -> torch.Tensor:
    """Rotary embedding, cache append and attention for one new token per row, one launch.

    ``q [M, H*D]``, ``k, v [M, Hkv*D]`` bf16 (rows may be strided views of one buffer), caches
    ``[M, Hkv, L, D]`` bf16 (the layout of transformers' ``StaticLayer``; slot ``position`` is
    written), ``cos, sin [L, D]`` bf16, ``mask [M, L]`` uint8, ``position`` an int64 device
    scalar (``per_row``: int64 ``[M]``, one slot per row).  Stands for ``apply_rotary_pos_emb``, ``Cache.update`` and the attention of
    ``LlamaAttention.forward`` (reached from ``vrl/models/families/janus_pro/policy.py:673-678``).
    ``lora`` is a :class:`LoraAdd` over exactly the q, k, v outputs passed here whose down-projection
    was launched: the attention then adds the up-projections itself (q, k, v stay as they are).
    ``out_lora`` is a :class:`LoraAdd` with one adapter over ``out`` built with ``parts = H``: the launch
    leaves that adapter's down-projection in its ``t``, one piece per head, for its ``launch_up``.
    ``split_workspace`` (from :func:`rope_attn_split_workspace`, without adapters): with at most 128
    (row, head) pairs several workgroups share the cached slots of a pair and the last one to finish
    merges their results (``vrl_rope_attn_decode_split_bf16``); launches over one workspace must not overlap.
    """
    dev = _require_device("k_cache", k_cache)
    if k_cache.dim() != 4 or k_cache.shape != v_cache.shape or k_cache.dtype != torch.bfloat16 or \
            v_cache.dtype != torch.bfloat16 or not k_cache.is_contiguous() or not v_cache.is_contiguous():
        raise ValueError("caches must be contiguous bfloat16 [M, Hkv, L, D] of one shape")
    M, Hkv, L, D = k_cache.shape
    for name, t in (("q", q), ("k", k), ("v", v)):
        if t.dtype != torch.bfloat16 or t.dim() != 2 or t.shape[0] != M or t.stride(1) != 1:
            raise ValueError(f"{name} must be bfloat16 [{M}, heads * {D}] with unit inner stride")
        if t.device != dev:
            raise ValueError(f"{name} is on {t.device}, expected {dev}")
    if q.shape[1] % D != 0 or tuple(k.shape) != (M, Hkv * D) or tuple(v.shape) != (M, Hkv * D) or \
            k.stride(0) != v.stride(0):
        raise ValueError("q must hold whole heads and k, v be [M, Hkv * D] with one row stride")
    H = q.shape[1] // D
    for name, t in (("cos", cos), ("sin", sin)):
        if t.dtype != torch.bfloat16 or tuple(t.shape) != (L, D) or not t.is_contiguous():
            raise ValueError(f"{name} must be contiguous bfloat16 [{L}, {D}]")
        _require_device(name, t, dev)
    if mask.dtype != torch.uint8 or tuple(mask.shape) != (M, L) or not mask.is_contiguous():
        raise ValueError(f"mask must be contiguous uint8 [{M}, {L}]")
    if position.dtype != torch.int64 or position.numel() != (M if per_row else 1) or not position.is_contiguous():
        raise ValueError("position must be an int64 tensor with one element (per_row: one per row)")
    for name, t in (("v_cache", v_cache), ("mask", mask), ("position", position)):
        _require_device(name, t, dev)
    if out is None:
        out = torch.empty((M, H * D), dtype=torch.bfloat16, device=dev)
    elif out.dtype != torch.bfloat16 or tuple(out.shape) != (M, H * D) or not out.is_contiguous():
        raise ValueError(f"out must be contiguous bfloat16 [{M}, {H * D}]")
    args = (q.data_ptr(), k.data_ptr(), v.data_ptr(), q.stride(0), k.stride(0), k_cache.data_ptr(),
            v_cache.data_ptr(), cos.data_ptr(), sin.data_ptr(), mask.data_ptr(), position.data_ptr(),
            out.data_ptr(), M, H, Hkv, D, L, float(scaling))
    record = lora.attn_record(q, k, v) if lora is not None else None
    if out_lora is not None:
        if out_lora.x.data_ptr() != out.data_ptr() or out_lora.parts != H:
            raise ValueError("out_lora must be built over `out` with one part per head")
        record = out_lora.attn_output_record(record)
    if split_workspace is not None:
        if record is not None:
            raise ValueError("the split form of the attention carries no adapters")
        need = _lib.load().vrl_rope_attn_decode_split_workspace_bytes(M, H, D)
        if split_workspace.dtype != torch.uint8 or split_workspace.numel() < need or \
                not split_workspace.is_contiguous() or split_workspace.device != dev:
            raise ValueError(f"split_workspace must be a contiguous uint8 tensor of {need} bytes on {dev}")
    if per_row and record is not None:
        record.position_per_row = 1
    with _on(dev):
        if per_row and record is None:   # one slot per row; the split form when a workspace is given
            rc = _lib.load().vrl_rope_attn_decode_rows_bf16(
                *args, split_workspace.data_ptr() if split_workspace is not None else None,
                split_workspace.numel() if split_workspace is not None else 0, _stream_handle(dev))
        elif split_workspace is not None:
            rc = _lib.load().vrl_rope_attn_decode_split_bf16(*args, split_workspace.data_ptr(),
                                                             split_workspace.numel(), _stream_handle(dev))
        elif record is None:
            rc = _lib.load().vrl_rope_attn_decode_bf16(*args, _stream_handle(dev))
        else:
            rc = _lib.load().vrl_rope_attn_decode_lora_bf16(*args, ctypes.byref(record), _stream_handle(dev))
    if rc and split_workspace is not None and not torch.cuda.is_current_stream_capturing():
        split_workspace.zero_()   # arrival counters a failed launch may have left above zero
    _lib.check(rc, "vrl_rope_attn_decode_bf16")
    return out


def rope_attn_split_workspace(M: int, H: int, D: int, device) -> torch.Tensor:
    """Zeroed scratch memory for the split form of :func:`rope_attn_decode` (counters, which every launch
    leaves at zero again, and the workgroups' partial results); one per stream of launches."""
    nbytes = _lib.load().vrl_rope_attn_decode_split_workspace_bytes(int(M), int(H), int(D))
    if nbytes == 0:
        raise ValueError("no split form for this shape")
    return torch.zeros(nbytes, dtype=torch.uint8, device=device)


class LoraAdd:
    """LoRA adapters added onto the outputs of int4 projections that share an input: two launches.

    ``adapters`` is a list of ``(A [r, K], B [N, r], scaling, y [M, N])`` with ``A``/``B`` the
    ``lora_A`` / ``lora_B`` weights of a PEFT wrapper (float32 or bfloat16, rank a multiple of 8 up
    to 64, kept by reference: an
    in-place weight sync is seen by the next launch) and ``y`` the bf16 output of the base
    projection, updated in place: ``y += scaling * (x A^T) B^T`` with the roundings the wrapper's
    own forward applies (``vrl/models/families/janus_pro/policy.py:298-324`` attaches the adapters).
    ``x`` is the fixed bf16 ``[M <= 32, K]`` input buffer of the group.

    ``parts > 1`` (one adapter only): the down-projection is left to the launch that produces ``x``, which
    writes it as ``parts`` partial rows per activation row (the attention launch does, one per head:
    :meth:`attn_output_record`); ``t`` is then ``[M, parts, r]`` and :meth:`launch_down` is not used.
    """

    def __init__(self, x: torch.Tensor, adapters, parts: int = 1):
        if x.dtype != torch.bfloat16 or x.dim() != 2 or not x.is_contiguous():
            raise ValueError("x must be contiguous bfloat16 [M, K]")
        dev = _require_device("x", x)
        M, K = x.shape
        if not 1 <= len(adapters) <= 4:
            raise ValueError("1 to 4 adapters per group")
        self.table = (_lib.LoraAdapter * len(adapters))()
        total = 0
        for rec, (A, B, scaling, y) in zip(self.table, adapters):
            if A.dtype != B.dtype or A.dtype not in (torch.float32, torch.bfloat16) or A.dtype != adapters[0][0].dtype:
                raise ValueError("adapter weights of one launch must all be float32 or all bfloat16")
            if A.dim() != 2 or B.dim() != 2 or A.shape[1] != K or B.shape[1] != A.shape[0] or \
                    not A.is_contiguous() or not B.is_contiguous():
                raise ValueError(f"adapter weights must be contiguous A [r, {K}] and B [N, r]")
            r, N = A.shape[0], B.shape[0]
            if y.dtype != torch.bfloat16 or tuple(y.shape) != (M, N) or not y.is_contiguous():
                raise ValueError(f"y must be contiguous bfloat16 [{M}, {N}]")
            for name, t in (("A", A), ("B", B), ("y", y)):
                _require_device(name, t, dev)
            rec.A, rec.B, rec.y, rec.N, rec.r = A.data_ptr(), B.data_ptr(), y.data_ptr(), N, r
            rec.scaling, rec.weights_fp32 = float(scaling), int(A.dtype == torch.float32)
            total += r
        if parts != 1 and (len(adapters) != 1 or not 1 < parts <= 256):
            raise ValueError("a down-projection in parts: one adapter, 2 to 256 parts")
        self.parts = int(parts)
        self.t = torch.empty((M, total) if parts == 1 else (M, parts, total), dtype=torch.float32, device=dev)
        self.x, self.M, self.K, self.device = x, M, K, dev
        self._keep = list(adapters)

    def launch_down(self):
        """``t = x . A^T`` for every adapter of the group."""
        with _on(self.device):
            rc = _lib.load().vrl_lora_down_bf16(self.x.data_ptr(), self.M, self.K, self.table, len(self.table),
                                                self.t.data_ptr(), _stream_handle(self.device))
        _lib.check(rc, "vrl_lora_down_bf16")

    def launch_up(self):
        """``y_i += scaling_i * t_i . B_i^T`` for every adapter of the group."""
        with _on(self.device):
            rc = _lib.load().vrl_lora_up_add_bf16(self.t.data_ptr(), self.parts, self.M, self.table,
                                                  len(self.table), _stream_handle(self.device))
        _lib.check(rc, "vrl_lora_up_add_bf16")

    def launch(self):
        self.launch_down()
        self.launch_up()

    def attn_record(self, q: torch.Tensor, k: torch.Tensor, v: torch.Tensor):
        """The ``vrl_attn_lora`` record that lets the attention launch add this group's up-projections
        to ``q``, ``k``, ``v`` (the outputs this group was built over; others have no adapter)."""
        rec = _lib.AttnLora()
        rec.t, rec.t_stride = self.t.data_ptr(), self.t.shape[1]
        rec.weights_fp32 = self.table[0].weights_fp32
        offset, found = 0, 0
        slots = {q.data_ptr(): 0, k.data_ptr(): 1, v.data_ptr(): 2}
        for ad in self.table:
            i = slots.get(ad.y)
            if i is None:
                raise ValueError("the adapter group holds an output that is not q, k or v of this call")
            setattr(rec, ("q_B", "k_B", "v_B")[i], ad.B)
            rec.r[i], rec.offset[i], rec.scaling[i] = ad.r, offset, ad.scaling
            offset += ad.r
            found += 1
        if not found:
            raise ValueError("no adapter")
        self._attn_record = rec   # kept alive for a launch that is only enqueued
        return rec

    def attn_output_record(self, rec=None):
        """Adds this group (one adapter over the attention output, built with ``parts = n_heads``) to a
        ``vrl_attn_lora`` record, or starts one: the attention launch then writes ``t`` itself."""
        if rec is None:
            rec = _lib.AttnLora()
            rec.weights_fp32 = self.table[0].weights_fp32
        elif rec.weights_fp32 != self.table[0].weights_fp32:
            raise ValueError("the adapters of one attention launch must all be float32 or all bfloat16")
        if len(self.table) != 1 or self.parts == 1 or self.K % self.parts != 0:
            raise ValueError("needs one adapter whose down-projection is split into one part per head")
        rec.o_A, rec.o_t, rec.o_r = self.table[0].A, self.t.data_ptr(), self.table[0].r
        self._attn_record = rec
        return rec
