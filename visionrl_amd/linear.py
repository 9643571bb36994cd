"""``Int4Linear``: drop-in for the bf16 ``nn.Linear`` layers of rollout decode.

The reference calls its decode linears as plain modules, ``module(x[..., K]) ->
[..., N]`` in the model dtype, under ``torch.no_grad()``
(``vrl/models/families/janus_pro/policy.py:673-678`` for the Llama trunk,
``policy.py:138-160`` for ``gen_head``).  These modules keep that calling
convention and route the arithmetic to the HIP library; the weights are frozen
(no gradient flows into the packed tensors).  A call whose input carries a gradient
(a train-time replay over the quantised base, e.g. under LoRA adapters) multiplies by
the dequantised weight through the library GEMM, so the gradient reaches the input.
"""

from __future__ import annotations

import weakref

import torch
import torch.nn.functional as F
from torch import nn

from . import ops
from .int4_format import check_packed, pack_nibbles, quantize_minmax

# Calls with more activation rows than this (the prompt pass) rebuild the bf16 weight (bit-exact
# tile, one launch) and hand the product to the library GEMM; the GEMV kernels are for decode.
GEMM_ROWS = 32


def _wants_grad(x: torch.Tensor) -> bool:
    """The HIP launches are not recorded by autograd: such calls take the dequant + GEMM route."""
    return torch.is_grad_enabled() and x.requires_grad


def _version(t: torch.Tensor):
    """The tensor's in-place modification counter, or ``None`` where torch keeps none (inference tensors)."""
    try:
        return t._version
    except RuntimeError:
        return None


def _source_state(*tensors):
    """What identifies the tensors a prepacked copy was made from: a weak reference to each, its
    modification counter and, for a tensor torch keeps no counter for (an inference tensor), the address
    and shape of its data instead.  In-place writes to such a tensor go unnoticed: ``prepack_()`` again
    after editing int4 buffers that were created under ``torch.inference_mode``."""
    return tuple((weakref.ref(t), _version(t), (t.data_ptr(), tuple(t.shape))) for t in tensors)


def _source_changed(state, *tensors) -> bool:
    for t, (ref, v0, where) in zip(tensors, state):
        if ref() is not t:
            return True
        if v0 is None:
            if (t.data_ptr(), tuple(t.shape)) != where:
                return True
        elif _version(t) != v0:
            return True
    return False


def _rows(x: torch.Tensor, in_features: int) -> torch.Tensor:
    if x.dtype != torch.bfloat16:
        raise TypeError(f"Int4Linear runs in bfloat16 like the policy it replaces, got {x.dtype}")
    if x.shape[-1] != in_features:
        raise ValueError(f"last dimension {x.shape[-1]} != in_features {in_features}")
    return x.reshape(-1, in_features).contiguous()


class Int4Linear(nn.Module):
    """int4 weight-only linear: ``y = x . dequant(qweight, scales, qzeros)^T (+ bias)``.

    Buffers (saved in ``state_dict``): ``qweight`` int32 ``[N, K/8]``, ``scales`` bf16
    ``[N, K/G]``, ``qzeros`` int32 ``[N, ceil(K/G/8)]``, optional ``bias`` bf16 ``[N]``.
    """

    def __init__(self, in_features: int, out_features: int, group_size: int = 128,
                 bias: bool = False, device=None):
        super().__init__()
        if group_size % 8 != 0 or in_features % group_size != 0:
            raise ValueError("group_size must be a multiple of 8 that divides in_features")
        self.in_features = int(in_features)
        self.out_features = int(out_features)
        self.group_size = int(group_size)
        groups = in_features // group_size
        self.register_buffer("qweight", torch.zeros((out_features, in_features // 8),
                                                    dtype=torch.int32, device=device))
        self.register_buffer("scales", torch.ones((out_features, groups), dtype=torch.bfloat16,
                                                  device=device))
        self.register_buffer("qzeros", torch.zeros((out_features, (groups + 7) // 8),
                                                   dtype=torch.int32, device=device))
        if bias:
            self.register_buffer("bias", torch.zeros(out_features, dtype=torch.bfloat16, device=device))
        else:
            self.bias = None

    @classmethod
    def from_packed(cls, qweight, scales, qzeros, group_size: int, bias=None) -> "Int4Linear":
        N, K, _ = check_packed(qweight, scales, qzeros, group_size)
        mod = cls(K, N, group_size, bias=bias is not None, device=qweight.device)
        mod.qweight, mod.scales, mod.qzeros = qweight.contiguous(), scales.contiguous(), qzeros.contiguous()
        if bias is not None:
            mod.bias = bias.detach().to(torch.bfloat16).contiguous()
        return mod

    @classmethod
    def from_linear(cls, linear: nn.Linear, group_size: int = 128) -> "Int4Linear":
        """Quantise an ``nn.Linear`` (min/max, asymmetric, per K-group) on its own device."""
        qweight, scales, qzeros = quantize_minmax(linear.weight.data, group_size)
        return cls.from_packed(qweight, scales, qzeros, group_size,
                               None if linear.bias is None else linear.bias.data)

    @classmethod
    def from_unpacked_zeros(cls, qweight, scales, zeros_u8, group_size: int, bias=None):
        """Accepts zero-points as an unpacked ``uint8 [N, K/G]`` tensor and packs them."""
        return cls.from_packed(qweight, scales, pack_nibbles(zeros_u8.to(torch.int32)), group_size, bias)

    def prepack_(self) -> "Int4Linear":
        """Keep a prepacked copy of the weight for decode-sized calls (a second copy in HBM).

        Calls with few activation rows then go through the plan-free launch over the
        MFMA-shaped blob; larger ones, and ``torch.compile``, keep using the canonical
        buffers, which stay the module's ``state_dict``.  No-op if the shape has no prepacked form.
        """
        self._packed = None
        if self.qweight.is_cuda and ops.PrepackedWeight.supported(self.out_features, self.in_features,
                                                                  self.group_size):
            self._packed = ops.int4_prepack(self.qweight, self.scales, self.qzeros, self.group_size)
            self._packed_from = _source_state(self.qweight, self.scales, self.qzeros)
            self._direct_rows = self._packed.direct_rows()
            self._call = ops.DirectCall([self._packed])
        group = getattr(self, "_group", None)
        if group is not None:  # rebuild the group's launch over the new copies
            self.group_with(*group[1:])
        leader = getattr(self, "_leader", None)
        leader = leader() if leader is not None else None   # the module whose launch computes this one's output too
        if leader is not None and leader is not self and getattr(leader, "_group", None) is not None:
            leader.group_with(*leader._group[1:])
        return self

    def packed_is_stale(self) -> bool:
        """True when the canonical buffers were written (``load_state_dict``, an in-place edit) or
        replaced (``.to()``) after :meth:`prepack_` copied them."""
        return getattr(self, "_packed", None) is not None and \
            _source_changed(self._packed_from, self.qweight, self.scales, self.qzeros)

    def _fresh_packed(self):
        """The prepacked copy, made again first if the canonical buffers changed under it."""
        packed = getattr(self, "_packed", None)
        if packed is not None and _source_changed(self._packed_from, self.qweight, self.scales, self.qzeros):
            if self.qweight.is_cuda and torch.cuda.is_current_stream_capturing():
                raise RuntimeError("the int4 weight changed after prepack_(): call prepack_() again before "
                                   "recording a graph over this module")
            self.prepack_()
            packed = self._packed
        return packed

    def group_with(self, *others: "Int4Linear") -> "Int4Linear":
        """Launch ``others`` together with this module whenever it is called (q|k|v of one layer).

        Modules that are applied to the same input one after the other, as
        ``LlamaAttention`` applies ``q_proj``, ``k_proj``, ``v_proj`` to ``hidden_states``
        (reached from ``vrl/models/families/janus_pro/policy.py:673-678``): a decode-sized call
        of this module computes all of them in one plan-free launch and hands each sibling its
        result, which the sibling returns when it is called with the very same tensor object
        next.  Needs ``prepack_()`` on every member; anything else falls back to one launch each.
        """
        if len(others) + 1 > ops.DirectGemv.MAX_PROBLEMS:
            raise ValueError(f"at most {ops.DirectGemv.MAX_PROBLEMS} modules per group")
        if any(o.in_features != self.in_features for o in others):
            raise ValueError("grouped modules take the same input")
        self._group = (self, *others)
        for m in others:
            m._leader = weakref.ref(self)
        self._group_call = None
        if all(getattr(m, "_packed", None) is not None for m in self._group):
            self._group_call = ops.DirectCall([m._packed for m in self._group])
        return self

    def dequantize(self) -> torch.Tensor:
        """The canonical bf16 weight ``[N, K]`` (bit-exact tile), e.g. for the train-time replay."""
        return ops.int4_dequant(self.qweight, self.scales, self.qzeros, self.group_size)

    def keep_dense_(self, keep: bool = True) -> "Int4Linear":
        """Keep the dequantised bf16 weight between calls (2 bytes per weight beside the 0.56 of the int4
        buffers): prompt-sized calls and the train-time replay (``policy.py:419-424``: one forward per
        micro-batch) then multiply by the kept tensor instead of rebuilding it every call.  It is rebuilt
        when the canonical buffers were written or replaced since; ``keep=False`` drops it."""
        self._keep_dense = bool(keep)
        self._dense = None
        return self

    def _dense_weight(self) -> torch.Tensor:
        """The bf16 weight for a library GEMM: the kept copy if there is one and it is current."""
        if not getattr(self, "_keep_dense", False):
            return ops.int4_dequant(self.qweight, self.scales, self.qzeros, self.group_size)
        kept = getattr(self, "_dense", None)
        if kept is None or _source_changed(kept[0], self.qweight, self.scales, self.qzeros):
            kept = (_source_state(self.qweight, self.scales, self.qzeros),
                    ops.int4_dequant(self.qweight, self.scales, self.qzeros, self.group_size))
            self._dense = kept
        return kept[1]

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        rows = _rows(x, self.in_features)
        handed = getattr(self, "_handed", None)
        if handed is not None:
            self._handed = None
        group = getattr(self, "_group", None)
        if group is not None:   # a new call of the leader: whatever it handed over before is void
            for m in group[1:]:
                m._handed = None
        if torch.compiler.is_compiling():
            y = ops.int4_gemv(rows, self.qweight, self.scales, self.qzeros, self.group_size)
        elif _wants_grad(x):
            y = F.linear(rows, self._dense_weight())
        elif handed is not None and handed[0] is x and handed[1] == _version(x):
            y = handed[2]   # computed by the group leader's launch from this very tensor, unchanged since
        else:  # eager decode: skip the operator dispatcher, it costs more than the kernel
            packed = self._fresh_packed()
            M = rows.shape[0]
            if packed is not None and packed.blob.device == rows.device:
                call = getattr(self, "_group_call", None)
                version = _version(x) if call is not None else None
                if call is not None and M <= call.max_rows and version is not None and \
                        not any(m.packed_is_stale() for m in group[1:]):
                    # (an input without a modification counter cannot be recognised later: no hand-over)
                    ys = call(rows)
                    for m, ym in zip(group[1:], ys[1:]):
                        m._handed = (x, version, ym)
                    y = ys[0]
                elif M <= self._direct_rows:
                    y = self._call(rows)[0]
                else:
                    packed = None
            else:
                packed = None
            if packed is None and M > GEMM_ROWS:
                # prompt-sized call: the GEMV kernels would stream the weight once per 16 rows
                y = F.linear(rows, self._dense_weight())
            elif packed is None:
                y = torch.empty((M, self.out_features), dtype=torch.bfloat16, device=rows.device)
                ops.int4_gemv_into(y, rows, self.qweight, self.scales, self.qzeros, self.group_size)
        if self.bias is not None:
            y = y + self.bias
        return y.reshape(*x.shape[:-1], self.out_features)

    def extra_repr(self) -> str:
        return (f"in_features={self.in_features}, out_features={self.out_features}, "
                f"group_size={self.group_size}, bias={self.bias is not None}")


class Int4GateUpSiLU(nn.Module):
    """Fused ``silu(gate_proj(x)) * up_proj(x)`` over one packed gate||up operand."""

    def __init__(self, gate: Int4Linear, up: Int4Linear):
        super().__init__()
        if (gate.in_features, gate.out_features, gate.group_size) != \
                (up.in_features, up.out_features, up.group_size):
            raise ValueError("gate_proj and up_proj must have the same shape and group size")
        if gate.bias is not None or up.bias is not None:
            raise ValueError("the fused gate/up operator takes bias-free projections")
        self.in_features = gate.in_features
        self.intermediate_size = gate.out_features
        self.group_size = gate.group_size
        self.register_buffer("qweight", torch.cat([gate.qweight, up.qweight], dim=0).contiguous())
        self.register_buffer("scales", torch.cat([gate.scales, up.scales], dim=0).contiguous())
        self.register_buffer("qzeros", torch.cat([gate.qzeros, up.qzeros], dim=0).contiguous())

    def prepack_(self) -> "Int4GateUpSiLU":
        """Keep a prepacked copy of gate||up for decode-sized calls (see ``Int4Linear.prepack_``)."""
        self._packed = None
        if self.qweight.is_cuda and self.intermediate_size % 16 == 0 and \
                ops.PrepackedWeight.supported(2 * self.intermediate_size, self.in_features, self.group_size):
            self._packed = ops.int4_prepack(self.qweight, self.scales, self.qzeros, self.group_size)
            self._packed_from = _source_state(self.qweight, self.scales, self.qzeros)
            self._direct_rows = self._packed.direct_rows(fused=True)
            self._call = ops.DirectCall([self._packed], fused=True)
        return self

    packed_is_stale = Int4Linear.packed_is_stale
    _fresh_packed = Int4Linear._fresh_packed
    keep_dense_ = Int4Linear.keep_dense_
    _dense_weight = Int4Linear._dense_weight

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        rows = _rows(x, self.in_features)
        packed = None if torch.compiler.is_compiling() else self._fresh_packed()
        grad = _wants_grad(x) and not torch.compiler.is_compiling()
        if packed is not None and not grad and not torch.compiler.is_compiling() \
                and rows.shape[0] <= self._direct_rows and packed.blob.device == rows.device:
            y = self._call(rows)[0]
        elif (grad or rows.shape[0] > GEMM_ROWS) and not torch.compiler.is_compiling():
            gate, up = F.linear(rows, self._dense_weight()).chunk(2, dim=-1)   # prompt-sized call: one library GEMM
            y = F.silu(gate) * up
        else:
            y = ops.int4_gate_up_silu(rows, self.qweight, self.scales, self.qzeros, self.group_size)
        return y.reshape(*x.shape[:-1], self.intermediate_size)


class Int4LlamaMLP(nn.Module):
    """``down_proj(silu(gate_proj(x)) * up_proj(x))`` with both halves in int4.

    Built from a Hugging Face ``LlamaMLP``-shaped module (attributes ``gate_proj``,
    ``up_proj``, ``down_proj``; SiLU activation).
    """

    def __init__(self, mlp: nn.Module, group_size: int = 128):
        super().__init__()
        act = getattr(mlp, "act_fn", None)
        if act is not None and not isinstance(act, nn.SiLU) and \
                getattr(act, "__name__", type(act).__name__).lower() not in ("silu", "siluactivation"):
            raise ValueError(f"fused MLP needs a SiLU activation, found {act!r}")
        as_int4 = lambda m: m if isinstance(m, Int4Linear) else Int4Linear.from_linear(m, group_size)
        self.gate_up = Int4GateUpSiLU(as_int4(mlp.gate_proj), as_int4(mlp.up_proj))
        self.down_proj = as_int4(mlp.down_proj)

    def prepack_(self) -> "Int4LlamaMLP":
        self.gate_up.prepack_()
        self.down_proj.prepack_()
        return self

    def keep_dense_(self, keep: bool = True) -> "Int4LlamaMLP":
        self.gate_up.keep_dense_(keep)
        self.down_proj.keep_dense_(keep)
        return self

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        return self.down_proj(self.gate_up(x))
