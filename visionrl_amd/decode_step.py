"""One decode step of an int4 Llama trunk as a fixed list of launches over static buffers.

The trunk call of a decode step (``vrl/models/families/janus_pro/policy.py:673-678``) runs the
Hugging Face ``LlamaModel`` on one new token per row: per layer some thirty small tensor ops
between the seven linears (norm in four ops, rotary in eight, cache update, mask building,
attention, residual adds).  At decode sizes every one of them is a launch that costs more than
the arithmetic in it.  :class:`NativeDecodeTrunk` runs the same layer as five launches:

    [add + RMSNorm ->] q|k|v (one int4 launch) -> rotary + cache append + attention -> o_proj
    -> [add + RMSNorm ->] gate|up + SiLU (one int4 launch) -> down_proj

where the residual add of the previous sublayer and the norm are applied by the int4 launch that
follows them while it stages its input (for hidden sizes up to 4096; a launch of their own
otherwise), over the same
``StaticCache`` tensors the prompt pass filled (``[rows, kv_heads, L_max, head_dim]``), the cache
slot of the new token held in device memory, and every buffer preallocated, so that the whole
step can be recorded as one HIP graph.  Arithmetic follows the library's roundings (each tensor
op in fp32, rounded to bf16); the attention keeps its probabilities in fp32.

Needs a trunk whose projections were swapped for prepacked :class:`Int4Linear` modules with the
fused MLP (``apply_int4_to_policy`` defaults) and carry no adapter; :meth:`NativeDecodeTrunk.unsupported`
says why a trunk does not qualify, and callers then keep the module path.
"""

from __future__ import annotations

import ctypes

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
        # the residual stream alternates between two buffers: a launch that adds to it reads one and
        # writes the other (its workgroups read the old stream while one of them writes the new one)
        streams = [new(hidden), new(hidden)]
        self.normed, self.attn = new(hidden), new(H * D)
        self._keep = [cache, cur, mask, slot, streams]
        lib = _lib.load()
        fuse_norm = hidden <= 4096   # the linears normalise their input while staging it
        calls = []       # (function, argument tuple without the stream)
        state = {"x": cur.view(rows, hidden), "res": None, "flip": 0}   # x: sublayer output not yet added to res

        def norm_weight(module):
            w = module.weight.data
            if w.dtype != torch.bfloat16 or tuple(w.shape) != (hidden,) or not w.is_contiguous():
                raise TypeError("norm weights must be contiguous bfloat16 [hidden]")
            self._keep.append(w)
            return w, float(module.variance_epsilon)

        def gemv(problems, norm=None):
            launch = ops.DirectGemv(problems, norm=norm)
            self._keep.append(launch)
            if norm is None:
                calls.append((lib.vrl_int4_gemv_prepacked_bf16, (launch.table, len(launch.table))))
            else:
                calls.append((lib.vrl_int4_gemv_prepacked_norm_bf16,
                              (launch.table, len(launch.table), ctypes.byref(launch.norm))))
            return launch.outputs

        def normed_gemv(module, weights, fused):
            """h = res + x; the linears over norm(h); afterwards res = h."""
            w, eps = norm_weight(module)
            h_out = streams[state["flip"]]
            state["flip"] ^= 1
            if fuse_norm:
                outs = gemv([(state["x"], pw, fused) for pw in weights], norm=(state["res"], w, eps, h_out))
            else:
                calls.append((lib.vrl_add_rmsnorm_bf16,
                              (state["x"].data_ptr(), state["res"].data_ptr() if state["res"] is not None else None,
                               w.data_ptr(), h_out.data_ptr(), self.normed.data_ptr(), rows, hidden, eps)))
                outs = gemv([(self.normed, pw, fused) for pw in weights])
            state["res"] = h_out
            return outs

        for i, layer in enumerate(trunk.layers):
            attn, mlp = layer.self_attn, layer.mlp
            q, k, v = normed_gemv(layer.input_layernorm,
                                  [attn.q_proj._packed, attn.k_proj._packed, attn.v_proj._packed], False)
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
            (state["x"],) = gemv([(self.attn, attn.o_proj._packed, False)])
            (act,) = normed_gemv(layer.post_attention_layernorm, [mlp.gate_up._packed], True)
            (state["x"],) = gemv([(act, mlp.down_proj._packed, False)])
        w, eps = norm_weight(trunk.norm)
        calls.append((lib.vrl_add_rmsnorm_bf16,
                      (state["x"].data_ptr(), state["res"].data_ptr(), w.data_ptr(),
                       streams[state["flip"]].data_ptr(), self.normed.data_ptr(), rows, hidden, eps)))
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
