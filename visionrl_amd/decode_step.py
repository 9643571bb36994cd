"""One decode step of an int4 Llama trunk as a fixed list of launches over static buffers.

The trunk call of a decode step (``vrl/models/families/janus_pro/policy.py:673-678``) runs the
Hugging Face ``LlamaModel`` on one new token per row: per layer some thirty small tensor ops
between the seven linears (norm in four ops, rotary in eight, cache update, mask building,
attention, residual adds).  At decode sizes every one of them is a launch that costs more than
the arithmetic in it.  :class:`NativeDecodeTrunk` runs the same layer as seven launches:

    add + RMSNorm -> q|k|v (one int4 launch) -> rotary + cache append + attention -> o_proj
    -> add + RMSNorm -> gate|up + SiLU (one int4 launch) -> down_proj

with the residual add of the previous sublayer folded into the next norm, over the same
``StaticCache`` tensors the prompt pass filled (``[rows, kv_heads, L_max, head_dim]``), the cache
slot of the new token held in device memory, and every buffer preallocated, so that the whole
step can be recorded as one HIP graph.  Arithmetic follows the library's roundings (each tensor
op in fp32, rounded to bf16); the attention keeps its probabilities in fp32.

Needs a trunk whose projections were swapped for prepacked :class:`Int4Linear` modules with the
fused MLP (``apply_int4_to_policy`` defaults) and carry no adapter; :meth:`NativeDecodeTrunk.unsupported`
says why a trunk does not qualify, and callers then keep the module path.
"""

from __future__ import annotations

import torch

from . import _lib, ops
from .linear import Int4Linear, Int4LlamaMLP

__all__ = ["NativeDecodeTrunk"]


def _plain_int4(module, name: str):
    if not isinstance(module, Int4Linear):
        raise TypeError(f"{name} is {type(module).__name__}, not a bare Int4Linear (adapters keep the module path)")
    if getattr(module, "_packed", None) is None:
        raise TypeError(f"{name} has no prepacked weight")
    if module.bias is not None:
        raise TypeError(f"{name} has a bias")
    return module._packed


class NativeDecodeTrunk:
    """``last_hidden_state`` of one new token per row, written into static buffers.

    ``cache`` is the ``StaticCache`` the prompt pass already went through (its per-layer ``keys`` /
    ``values`` tensors are appended to in place), ``cur`` the ``[rows, 1, hidden]`` input embedding
    buffer, ``mask`` a uint8 ``[rows, L_max]`` buffer (0 = padding slot), ``slot`` an int64 device
    scalar holding the cache slot the new token takes; :meth:`run` leaves ``slot`` untouched.
    """

    @staticmethod
    def unsupported(trunk, rows: int, max_len: int) -> str | None:
        """Why this trunk cannot run natively at ``rows`` rows, or ``None`` if it can."""
        try:
            conf = trunk.config
            head_dim = getattr(conf, "head_dim", None) or conf.hidden_size // conf.num_attention_heads
            if head_dim not in (64, 128):
                return f"head_dim {head_dim} (64 or 128)"
            if max_len > 8192:
                return f"cache length {max_len} > 8192"
            if conf.hidden_size % 8 != 0 or conf.hidden_size > 16384:
                return f"hidden size {conf.hidden_size}"
            for i, layer in enumerate(trunk.layers):
                attn, mlp = layer.self_attn, layer.mlp
                packed = [_plain_int4(getattr(attn, n), f"layers[{i}].self_attn.{n}")
                          for n in ("q_proj", "k_proj", "v_proj", "o_proj")]
                if not isinstance(mlp, Int4LlamaMLP) or getattr(mlp.gate_up, "_packed", None) is None:
                    return f"layers[{i}].mlp is not a prepacked fused int4 MLP"
                packed.append(_plain_int4(mlp.down_proj, f"layers[{i}].mlp.down_proj"))
                if rows > min(w.direct_rows(False, 3) for w in packed[:3]) or \
                        rows > min(w.direct_rows() for w in packed[3:]) or \
                        rows > mlp.gate_up._packed.direct_rows(True):
                    return f"{rows} rows exceed what one plan-free launch takes"
        except (AttributeError, TypeError) as exc:
            return str(exc)
        return None

    def __init__(self, trunk, cache, cur: torch.Tensor, mask: torch.Tensor, slot: torch.Tensor):
        rows, one, hidden = cur.shape
        why = self.unsupported(trunk, rows, mask.shape[1])
        if why is not None:
            raise TypeError(f"trunk cannot run natively: {why}")
        if one != 1 or cur.dtype != torch.bfloat16 or not cur.is_cuda or not cur.is_contiguous():
            raise ValueError("cur must be a contiguous bfloat16 [rows, 1, hidden] device buffer")
        if mask.dtype != torch.uint8 or mask.shape[0] != rows or not mask.is_contiguous():
            raise ValueError("mask must be contiguous uint8 [rows, L_max]")
        if slot.dtype != torch.int64 or slot.numel() != 1:
            raise ValueError("slot must be an int64 device scalar")
        dev = cur.device
        conf = trunk.config
        self.device, self.rows, self.hidden, self.max_len = dev, rows, hidden, mask.shape[1]
        H, Hkv = conf.num_attention_heads, conf.num_key_value_heads
        D = getattr(conf, "head_dim", None) or hidden // H
        if len(cache.layers) != len(trunk.layers) or not all(l.is_initialized for l in cache.layers):
            raise ValueError("the cache must have gone through the prompt pass of this trunk")
        # rotary tables straight from the model's own module: row p is what it returns for position p
        with torch.no_grad():
            cos, sin = trunk.rotary_emb(cur, position_ids=torch.arange(self.max_len, device=dev)[None])
        self.cos, self.sin = cos[0].contiguous(), sin[0].contiguous()
        new = lambda n: torch.empty((rows, n), dtype=torch.bfloat16, device=dev)
        self.h, self.normed, self.attn = new(hidden), new(hidden), new(H * D)
        self._keep = [cache, cur, mask, slot]
        lib = _lib.load()
        x2d = cur.view(rows, hidden)
        calls = []   # (function, argument tuple without the stream)
        pending = None   # output of the previous sublayer, still to be added to the residual stream

        def norm(module, x, residual):
            w = module.weight.data
            if w.dtype != torch.bfloat16 or tuple(w.shape) != (hidden,):
                raise TypeError("norm weights must be bfloat16 [hidden]")
            self._keep.append(w)
            calls.append((lib.vrl_add_rmsnorm_bf16, (x.data_ptr(), residual.data_ptr() if residual is not None else None,
                                                     w.data_ptr(), self.h.data_ptr(), self.normed.data_ptr(),
                                                     rows, hidden, float(module.variance_epsilon))))

        def gemv(problems):
            launch = ops.DirectGemv(problems)
            self._keep.append(launch)
            calls.append((lib.vrl_int4_gemv_prepacked_bf16, (launch.table, len(launch.table))))
            return launch.outputs

        for i, layer in enumerate(trunk.layers):
            attn, mlp = layer.self_attn, layer.mlp
            norm(layer.input_layernorm, x2d if pending is None else pending, None if pending is None else self.h)
            q, k, v = gemv([(self.normed, attn.q_proj._packed, False), (self.normed, attn.k_proj._packed, False),
                            (self.normed, attn.v_proj._packed, False)])
            if q.shape[1] != H * D or k.shape[1] != Hkv * D or v.shape[1] != Hkv * D:
                raise TypeError(f"layers[{i}] projections do not match the attention geometry")
            keys, values = cache.layers[i].keys, cache.layers[i].values
            if tuple(keys.shape) != (rows, Hkv, self.max_len, D) or keys.dtype != torch.bfloat16 or \
                    not keys.is_contiguous() or not values.is_contiguous():
                raise ValueError(f"cache layer {i} is not bfloat16 [rows, kv_heads, L_max, head_dim]")
            calls.append((lib.vrl_rope_attn_decode_bf16,
                          (q.data_ptr(), k.data_ptr(), v.data_ptr(), q.stride(0), k.stride(0), keys.data_ptr(),
                           values.data_ptr(), self.cos.data_ptr(), self.sin.data_ptr(), mask.data_ptr(),
                           slot.data_ptr(), self.attn.data_ptr(), rows, H, Hkv, D, self.max_len,
                           float(attn.scaling))))
            (o,) = gemv([(self.attn, attn.o_proj._packed, False)])
            norm(layer.post_attention_layernorm, o, self.h)
            (act,) = gemv([(self.normed, mlp.gate_up._packed, True)])
            (pending,) = gemv([(act, mlp.down_proj._packed, False)])
        norm(trunk.norm, pending, self.h)
        self._calls = calls
        self.launches = len(calls)

    def run(self) -> torch.Tensor:
        """Enqueue the step on the current stream; returns the ``[rows, hidden]`` output buffer."""
        stream = torch.cuda.current_stream(self.device).cuda_stream
        with ops._on(self.device):
            for fn, args in self._calls:
                rc = fn(*args, stream)
                if rc:
                    _lib.check(rc, fn.__name__)
        return self.normed
