"""One decode step of an int4 Llama trunk as a fixed list of launches over static buffers.

The trunk call of a decode step (``vrl/models/families/janus_pro/policy.py:673-678``) runs the
Hugging Face ``LlamaModel`` on one new token per row: per layer some thirty small tensor ops
between the seven linears (norm in four ops, rotary in eight, cache update, mask building,
attention, residual adds).  At decode sizes every one of them is a launch that costs more than
the arithmetic in it.  :class:`NativeDecodeTrunk` runs the same layer as five launches:

    [add + RMSNorm ->] q|k|v (one int4 launch) -> rotary + cache append + attention -> o_proj
    -> [add + RMSNorm ->] gate|up + SiLU (one int4 launch) -> down_proj

where the norm is applied by the int4 launch that follows it while it stages its input, and the
residual add by the launch that produces the sublayer's output as it stores (hidden sizes up to
4096; above that, and for rows wider than 2048 at more than 16 rows, add and norm are a launch of
their own: measured faster there), over the same
``StaticCache`` tensors the prompt pass filled (``[rows, kv_heads, L_max, head_dim]``), the cache
slot of the new token held in device memory, and every buffer preallocated, so that the whole
step can be recorded as one HIP graph.  Arithmetic follows the library's roundings (each tensor
op in fp32, rounded to bf16); the attention keeps its probabilities in fp32.

Needs a trunk whose projections were swapped for prepacked :class:`Int4Linear` modules with the
fused MLP (``apply_int4_to_policy`` defaults).  Attention projections may carry one active LoRA
adapter each (the reference's default, ``policy.py:81-88``, ``:298-324``): their layer then takes
the norm as a launch of its own (the adapters read the normalised row) when the rows are wider than
2048 values or more than 8: six launches; otherwise the adapters' workgroups of the q|k|v launch
normalise the rows themselves (up to 8 rows).  The
down-projections of the q|k|v adapters ride with the q|k|v launch as extra workgroups and their
up-projections are added by the attention launch as it reads q, k, v; the attention launch also leaves
o_proj's down-projection behind, one piece per head, and o_proj's launch adds the up-projection before
it stores.  :meth:`NativeDecodeTrunk.unsupported` says why a trunk does not
qualify, and callers then keep the module path.
"""

from __future__ import annotations

import ctypes

import torch

from . import _lib, ops
from .linear import Int4Linear, Int4LlamaMLP

__all__ = ["NativeDecodeTrunk", "trunk_signature"]


def _plain_int4(module, name: str):
    if not isinstance(module, Int4Linear):
        raise TypeError(f"{name} is {type(module).__name__}, not a bare Int4Linear (adapters keep the module path)")
    if getattr(module, "_packed", None) is None:
        raise TypeError(f"{name} has no prepacked weight")
    if module.bias is not None:
        raise TypeError(f"{name} has a bias")
    return module._packed


def _adapter_of(module, name: str):
    """``(A, B, scaling)`` of the one active LoRA adapter of a PEFT-style wrapper.

    Reads the attributes of peft's ``lora.Linear`` (``lora_A`` / ``lora_B`` module dicts keyed by
    adapter name, ``scaling``, ``active_adapters``, ``merged``, ``disable_adapters``, ``use_dora``;
    the wrappers ``policy.py:298-324`` attaches); a plain pair of linears with a float
    ``scaling`` attribute is taken too.  The weights are returned by reference, so an in-place
    weight sync reaches the launches that hold them.
    """
    if getattr(module, "merged", False) or getattr(module, "disable_adapters", False):
        raise TypeError(f"{name}: merged or disabled adapters")
    lora_a, lora_b, scaling = module.lora_A, module.lora_B, getattr(module, "scaling", 1.0)
    if hasattr(lora_a, "keys"):
        active = getattr(module, "active_adapters", None) or getattr(module, "active_adapter", "default")
        active = [active] if isinstance(active, str) else list(active)
        active = [key for key in active if key in lora_a]
        if len(active) != 1:
            raise TypeError(f"{name}: exactly one active adapter is supported, found {active}")
        key = active[0]
        if getattr(module, "use_dora", None) and module.use_dora.get(key):
            raise TypeError(f"{name}: DoRA adapters keep the module path")
        drop = getattr(module, "lora_dropout", None)
        drop = drop[key] if drop is not None and key in drop else None
        if isinstance(drop, torch.nn.Dropout) and drop.p > 0 and drop.training:
            raise TypeError(f"{name}: adapter dropout is active")
        lora_a, lora_b = lora_a[key], lora_b[key]
        scaling = scaling[key] if hasattr(scaling, "keys") else scaling
    if getattr(lora_a, "bias", None) is not None or getattr(lora_b, "bias", None) is not None:
        raise TypeError(f"{name}: adapter linears with a bias")
    A, B = lora_a.weight.data, lora_b.weight.data
    if A.dtype != B.dtype or A.dtype not in (torch.float32, torch.bfloat16):
        raise TypeError(f"{name}: adapter weights must both be float32 or both bfloat16")
    if A.shape[0] % 8 != 0 or A.shape[0] > 64 or not A.is_contiguous() or not B.is_contiguous():
        raise TypeError(f"{name}: adapter rank {A.shape[0]} (a multiple of 8 up to 64)")
    return A, B, float(scaling)


def _projection(module, name: str):
    """``(prepacked weight, adapter or None)`` of a bare int4 projection or a LoRA wrapper around one."""
    if isinstance(module, Int4Linear):
        return _plain_int4(module, name), None
    base = getattr(module, "base_layer", None)
    if not isinstance(base, Int4Linear) or not hasattr(module, "lora_A") or not hasattr(module, "lora_B"):
        raise TypeError(f"{name} is {type(module).__name__}: neither an Int4Linear nor a LoRA wrapper around one")
    return _plain_int4(base, name + ".base_layer"), _adapter_of(module, name)


def trunk_signature(trunk) -> tuple:
    """What a recorded decode step bakes in besides tensor addresses: which module objects serve the
    projections and the state of their adapters (merged, disabled, active names, scaling).  A
    recorded step or a native launch list is valid while this value is unchanged; weight values may
    change in place."""
    sig = []
    for layer in trunk.layers:
        for owner, names in ((layer.self_attn, ("q_proj", "k_proj", "v_proj", "o_proj")), (layer, ("mlp",))):
            for name in names:
                mod = getattr(owner, name, None)
                active = getattr(mod, "active_adapters", None) or getattr(mod, "active_adapter", None)
                active = tuple(active) if isinstance(active, (list, tuple)) else active
                scaling = getattr(mod, "scaling", None)
                scaling = tuple(sorted(scaling.items())) if hasattr(scaling, "items") else scaling
                sig.append((id(mod), bool(getattr(mod, "merged", False)),
                            bool(getattr(mod, "disable_adapters", False)), active, scaling, _packed_ids(mod)))
    return tuple(sig)


def _packed_ids(mod) -> tuple:
    """The prepacked copies a projection (or fused MLP) streams from, made again first where the canonical
    buffers changed since (``load_state_dict`` into a prepacked module): a launch list holds blob
    addresses, so a new copy is a new signature."""
    inner = getattr(mod, "base_layer", mod)
    parts = (inner.gate_up, inner.down_proj) if isinstance(inner, Int4LlamaMLP) else (inner,)
    out = []
    for part in parts:
        fresh = getattr(part, "_fresh_packed", None)
        out.append(id(fresh()) if fresh is not None else None)
    return tuple(out)


class NativeDecodeTrunk:
    """``last_hidden_state`` of one new token per row, written into static buffers.

    ``cache`` is the ``StaticCache`` the prompt pass already went through (its per-layer ``keys`` /
    ``values`` tensors are appended to in place), ``cur`` the ``[rows, 1, hidden]`` input embedding
    buffer, ``mask`` a uint8 ``[rows, L_max]`` buffer (0 = padding slot), ``slot`` an int64 device
    scalar holding the cache slot the new token takes, or an int64 ``[rows]`` tensor with one slot per
    row (rows that advance at different times); :meth:`run` leaves ``slot`` untouched.
    """

    ROW_BLOCK = 32               # rows one plan-free launch takes; more rows go as several launches per linear,
    MAX_ROWS = 64                # each reading the weights again (beyond this a dequantised GEMM is the better form)
    SPLIT_ATTENTION_FROM = 512   # cache slots from which the attention of few rows runs in its split form
    SPLIT_ATTENTION_FROM_TWO = 768   # ... where the library gives a pair two workgroups (65 to 128 pairs)
    SPLIT_ATTENTION_PAIRS = 128  # (row, head) pairs up to which the library splits a pair's slots

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
                packed = [_projection(getattr(attn, n), f"layers[{i}].self_attn.{n}")[0]
                          for n in ("q_proj", "k_proj", "v_proj", "o_proj")]
                if not isinstance(mlp, Int4LlamaMLP) or getattr(mlp.gate_up, "_packed", None) is None:
                    return f"layers[{i}].mlp is not a prepacked fused int4 MLP"
                packed.append(_plain_int4(mlp.down_proj, f"layers[{i}].mlp.down_proj"))
                block = min(rows, NativeDecodeTrunk.ROW_BLOCK)   # more rows go as several launches per linear
                if rows > NativeDecodeTrunk.MAX_ROWS or \
                        block > min(w.direct_rows(False, 3) for w in packed[:3]) or \
                        block > min(w.direct_rows() for w in packed[3:]) or \
                        block > mlp.gate_up._packed.direct_rows(True):
                    return f"{rows} rows exceed what the plan-free launches take"
                if rows > NativeDecodeTrunk.ROW_BLOCK and any(
                        _projection(getattr(attn, n), n)[1] is not None for n in ("q_proj", "k_proj", "v_proj", "o_proj")):
                    return f"{rows} rows with adapters (their launches take up to {NativeDecodeTrunk.ROW_BLOCK})"
        except (AttributeError, TypeError) as exc:
            return str(exc)
        return None

    def __init__(self, trunk, cache, cur: torch.Tensor, mask: torch.Tensor, slot: torch.Tensor,
                 final_norm: bool = True):
        """``final_norm=False`` (hidden sizes up to 4096) leaves the model's last norm to the launch that
        consumes the step's output: :attr:`final` then holds ``(x, residual, norm weight, eps)`` for a
        launch that normalises while it stages its input, and :meth:`run` returns ``None``."""
        rows, one, hidden = cur.shape
        why = self.unsupported(trunk, rows, mask.shape[1])
        if why is not None:
            raise TypeError(f"trunk cannot run natively: {why}")
        if one != 1 or cur.dtype != torch.bfloat16 or not cur.is_cuda or not cur.is_contiguous():
            raise ValueError("cur must be a contiguous bfloat16 [rows, 1, hidden] device buffer")
        if mask.dtype != torch.uint8 or mask.shape[0] != rows or not mask.is_contiguous():
            raise ValueError("mask must be contiguous uint8 [rows, L_max]")
        if slot.dtype != torch.int64 or slot.numel() not in (1, rows) or not slot.is_contiguous():
            raise ValueError("slot must be an int64 device scalar, or one slot per row")
        per_row = slot.numel() != 1   # rows that advance at different times (a scheduler's partial batches)
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
        # writes the other (the input embedding is the first stream and must stay as it is; a normalising
        # launch's workgroups read the old stream while one of them writes the new one)
        streams = [new(hidden), new(hidden)]
        self.normed, self.attn = new(hidden), new(H * D)
        self._keep = [cache, cur, mask, slot, streams]
        lib = _lib.load()
        # The linears normalise their input while staging it, where that is the faster form: every workgroup of
        # such a launch normalises all the rows it stages, which for wide rows and many of them costs more than
        # a norm launch of its own in front of a launch that reads every weight once (hidden 4096: q|k|v 30.0
        # against 2.9 + 14.6 us at 32 rows; at 16 rows the two forms tie, below that and at hidden 2048 the
        # fused form wins).  That norm launch then adds the residual stream as well.
        fuse_norm = hidden <= 4096 and (hidden <= 2048 or rows <= 16)
        # With few (row, head) pairs and a cache that grows long the attention divides a pair's cached slots
        # over several workgroups (one workspace for all layers: the launches are ordered by the stream).
        # Its exchange costs about 1.5 us per launch, which pays from about 500 cached slots on (at 2 rows a
        # step takes 0.85 / 0.86 / 0.86 / 0.88 ms at 450 / 530 / 610 / 830 slots against 0.82 / 0.86 / 0.91 /
        # 0.96 ms); the launch is recorded once for a whole generation, and while a row has fewer than 512
        # slots filled it leaves each of the row's pairs to one workgroup, as the other form does.
        # (the library's own lines: 512 slots with 8 or 4 workgroups per pair, 768 with two, where half the
        # compute units are busy without the split: 1.07 against 1.03 ms per step at 8 rows and 580 slots)
        self._split_from = self.SPLIT_ATTENTION_FROM if rows * H <= 64 else self.SPLIT_ATTENTION_FROM_TWO
        split_ws = ops.rope_attn_split_workspace(rows, H, D, dev) \
            if rows * H <= self.SPLIT_ATTENTION_PAIRS and self.max_len >= self._split_from else None
        self._keep.append(split_ws)
        self._split_ws = split_ws
        calls = []       # (function, argument tuple without the stream)
        short_form = []  # (index, call): the one-workgroup attention launches that stand in while the cache is short
        state = {"x": cur.view(rows, hidden), "res": None, "flip": 0}   # x: sublayer output not yet added to res

        def norm_weight(module):
            w = module.weight.data
            if w.dtype != torch.bfloat16 or tuple(w.shape) != (hidden,) or not w.is_contiguous():
                raise TypeError("norm weights must be contiguous bfloat16 [hidden]")
            self._keep.append(w)
            return w, float(module.variance_epsilon)

        blocks = [(r0, min(rows, r0 + self.ROW_BLOCK)) for r0 in range(0, rows, self.ROW_BLOCK)]

        def gemv(problems, norm=None, joins=None):
            """The launches of one linear group over all rows: one per block of ROW_BLOCK rows."""
            cut = lambda t, r0, r1: None if t is None else (t if len(blocks) == 1 else t[r0:r1])
            if joins is not None:
                # the sublayer's output joins the residual stream in the launch that produces it
                # (`hidden_states = residual + hidden_states`): the next norm then reads one tensor
                (x, pw, _), = problems
                out = streams[state["flip"]]
                state["flip"] ^= 1
                for r0, r1 in blocks:
                    launch = ops.EpilogueGemv(cut(x, r0, r1), pw, residual=cut(joins, r0, r1), out=cut(out, r0, r1))
                    self._keep.append(launch)
                    calls.append((lib.vrl_int4_gemv_prepacked_epilogue_bf16,
                                  (launch._gemv.table, None, ctypes.byref(launch.epilogue))))
                return [out]
            outs = [new(pw.N // 2 if fused else pw.N) for _, pw, fused in problems] if len(blocks) > 1 else None
            for r0, r1 in blocks:
                xs = {}   # one view per input tensor and block: a normalising launch wants the same object for all
                part = [(xs.setdefault(id(x), cut(x, r0, r1)), pw, fused) for x, pw, fused in problems]
                launch = ops.DirectGemv(part, outputs=None if outs is None else [y[r0:r1] for y in outs],
                                        norm=None if norm is None else
                                        (cut(norm[0], r0, r1), norm[1], norm[2], cut(norm[3], r0, r1)))
                self._keep.append(launch)
                if norm is None:
                    calls.append((lib.vrl_int4_gemv_prepacked_bf16, (launch.table, len(launch.table))))
                else:
                    calls.append((lib.vrl_int4_gemv_prepacked_norm_bf16,
                                  (launch.table, len(launch.table), ctypes.byref(launch.norm))))
                if outs is None:
                    outs = launch.outputs
            return outs

        def lora(x, outs, adapters, up=True, down=True, parts=1):
            """outs[i] += adapter i applied to x, for the projections that carry one: a down-projection
            launch (unless another launch computes it: ``down=False``, or the producer of x leaves it in
            ``parts`` pieces, as the attention does for its output) and, unless the consumer adds the
            up-projection itself (``up=False``: the attention does for q, k, v), an up-projection
            launch.  Returns the group or ``None``."""
            todo = [(A, B, s, y) for y, ad in zip(outs, adapters) if ad is not None for A, B, s in [ad]]
            if not todo:
                return None
            launch = ops.LoraAdd(x, todo, parts=parts)
            self._keep.append(launch)
            n = len(launch.table)
            if down and parts == 1:
                calls.append((lib.vrl_lora_down_bf16, (x.data_ptr(), rows, x.shape[1], launch.table, n,
                                                       launch.t.data_ptr())))
            if up:
                calls.append((lib.vrl_lora_up_add_bf16, (launch.t.data_ptr(), parts, rows, launch.table, n)))
            return launch

        def normed_gemv(module, weights, fused, adapters=(), up=True):
            """h = res + x (h = x where x already holds the stream); the linears over norm(h); afterwards res = h.
            Returns (outputs, adapter group)."""
            w, eps = norm_weight(module)
            h_out = None
            if state["res"] is not None:
                h_out = streams[state["flip"]]
                state["flip"] ^= 1
            group = None
            with_adapters = any(ad is not None for ad in adapters)
            if fuse_norm and not with_adapters:
                outs = gemv([(state["x"], pw, fused) for pw in weights], norm=(state["res"], w, eps, h_out))
            elif fuse_norm and not fused and hidden <= 2048 and rows <= 8:
                # rows of up to 2048 values, at most 8 of them: the adapters' down-projection workgroups of the
                # q|k|v launch normalise the rows themselves, so the layer needs no norm launch of its own here
                # either (7.7 against 3.5 + 6.0 us at 2 rows; a step with adapters, same box, alternating:
                # 0.98-1.00 against 1.00-1.02 ms at B=1, 1.11 against 1.13-1.16 ms at B=4; with 16 rows those
                # workgroups become the launch's longest, 1.34 against 1.29 ms at B=8, and at 32 rows they hold
                # more rows than their registers take)
                launch_at = len(calls)
                outs = gemv([(state["x"], pw, fused) for pw in weights], norm=(state["res"], w, eps, h_out))
                group = lora(state["x"], outs, adapters, up, down=False)
                calls[launch_at] = (lib.vrl_int4_gemv_prepacked_norm_lora_bf16,
                                    (*calls[launch_at][1], group.table, len(group.table), group.t.data_ptr()))
            else:
                calls.append((lib.vrl_add_rmsnorm_bf16,
                              (state["x"].data_ptr(), state["res"].data_ptr() if state["res"] is not None else None,
                               w.data_ptr(), h_out.data_ptr() if h_out is not None else None,
                               self.normed.data_ptr(), rows, hidden, eps)))
                # the adapters read the normalised row, so it is written out; their down-projection and the
                # base projections share one launch
                launch_at = len(calls)
                outs = gemv([(self.normed, pw, fused) for pw in weights])
                group = lora(self.normed, outs, adapters, up, down=fused)
                if group is not None and not fused:
                    calls[launch_at] = (lib.vrl_int4_gemv_prepacked_lora_bf16,
                                        (*calls[launch_at][1], group.table, len(group.table), group.t.data_ptr()))
            state["res"] = h_out if h_out is not None else state["x"]
            return outs, group

        for i, layer in enumerate(trunk.layers):
            attn, mlp = layer.self_attn, layer.mlp
            proj = {n: _projection(getattr(attn, n), f"layers[{i}].self_attn.{n}")
                    for n in ("q_proj", "k_proj", "v_proj", "o_proj")}
            (q, k, v), group = normed_gemv(layer.input_layernorm,
                                           [proj[n][0] for n in ("q_proj", "k_proj", "v_proj")], False,
                                           [proj[n][1] for n in ("q_proj", "k_proj", "v_proj")], up=False)
            if q.shape[1] != H * D or k.shape[1] != Hkv * D or v.shape[1] != Hkv * D:
                raise TypeError(f"layers[{i}] projections do not match the attention geometry")
            keys, values = cache.layers[i].keys, cache.layers[i].values
            if tuple(keys.shape) != (rows, Hkv, self.max_len, D) or keys.dtype != torch.bfloat16 or \
                    not keys.is_contiguous() or not values.is_contiguous():
                raise ValueError(f"cache layer {i} is not bfloat16 [rows, kv_heads, L_max, head_dim]")
            attn_args = (q.data_ptr(), k.data_ptr(), v.data_ptr(), q.stride(0), k.stride(0), keys.data_ptr(),
                         values.data_ptr(), self.cos.data_ptr(), self.sin.data_ptr(), mask.data_ptr(),
                         slot.data_ptr(), self.attn.data_ptr(), rows, H, Hkv, D, self.max_len, float(attn.scaling))
            # the attention adds the up-projections of the q, k, v adapters while it reads them, and leaves
            # the down-projection of o_proj's adapter behind, one piece per head
            record = group.attn_record(q, k, v) if group is not None else None
            attn_at = len(calls)
            calls.append(None)
            launch_at = len(calls)
            # o_proj's output joins the residual stream in its own launch, unless an adapter's launch form stores it
            joins = state["res"] if proj["o_proj"][1] is None and fuse_norm else None
            outs = gemv([(self.attn, proj["o_proj"][0], False)], joins=joins)
            if joins is not None:
                state["res"] = None
            o_group = lora(self.attn, outs, [proj["o_proj"][1]], up=False, parts=H)
            if o_group is not None:   # o_proj's launch adds the up-projection itself
                record = o_group.attn_output_record(record)
                calls[launch_at] = (lib.vrl_int4_gemv_prepacked_lora_up_bf16,
                                    (calls[launch_at][1][0], o_group.table, o_group.t.data_ptr(), H))
            if record is not None:
                record.position_per_row = 1 if per_row else 0
                calls[attn_at] = (lib.vrl_rope_attn_decode_lora_bf16, (*attn_args, ctypes.byref(record)))
            elif per_row:
                calls[attn_at] = (lib.vrl_rope_attn_decode_rows_bf16,
                                  (*attn_args, split_ws.data_ptr() if split_ws is not None else None,
                                   split_ws.numel() if split_ws is not None else 0))
            elif split_ws is not None:
                calls[attn_at] = (lib.vrl_rope_attn_decode_split_bf16,
                                  (*attn_args, split_ws.data_ptr(), split_ws.numel()))
                short_form.append((attn_at, (lib.vrl_rope_attn_decode_bf16, attn_args)))
            else:
                calls[attn_at] = (lib.vrl_rope_attn_decode_bf16, attn_args)
            (state["x"],) = outs
            (act,), _ = normed_gemv(layer.post_attention_layernorm, [mlp.gate_up._packed], True)
            (state["x"],) = gemv([(act, mlp.down_proj._packed, False)], joins=state["res"] if fuse_norm else None)
            if fuse_norm:
                state["res"] = None
        w, eps = norm_weight(trunk.norm)
        self.final = None
        if final_norm or hidden > 4096:
            res = state["res"]
            calls.append((lib.vrl_add_rmsnorm_bf16,
                          (state["x"].data_ptr(), res.data_ptr() if res is not None else None, w.data_ptr(),
                           streams[state["flip"]].data_ptr() if res is not None else None,
                           self.normed.data_ptr(), rows, hidden, eps)))
        else:
            self.final = (state["x"], state["res"], w, eps)
            self.normed = None
        self._calls = calls
        self.launches = len(calls)
        # the same list as records of the library's own walk over it: one host call per step
        self._table = _lib.step_calls(calls)
        # The split launches leave a row with fewer than SPLIT_ATTENTION_FROM cached slots to one workgroup per
        # pair themselves, but the workgroups that then have nothing to do still cost about 1 us per launch
        # (7.2 against 6.2 us at 150 slots, 9.0 against 7.8 at 330).  A caller that knows on the host how far
        # the rows have come (the sampling loop does) asks for the list with the one-workgroup launches instead.
        self._calls_short = self._table_short = None
        if short_form:
            self._calls_short = list(calls)
            for at, call in short_form:
                self._calls_short[at] = call
            self._table_short = _lib.step_calls(self._calls_short)
        self._failed_at = ctypes.c_int(-1)

    def short_form(self, cached_slots: int) -> bool:
        """Whether :meth:`run` has a launch list of its own for a step that finds ``cached_slots`` filled slots
        (the most any row holds): the split attention's one-workgroup stand-in below ``SPLIT_ATTENTION_FROM``
        (``SPLIT_ATTENTION_FROM_TWO`` for 65 to 128 pairs)."""
        return self._table_short is not None and 0 <= cached_slots < self._split_from

    def run(self, short: bool = False) -> torch.Tensor:
        """Enqueue the step on the current stream; returns the ``[rows, hidden]`` output buffer.  ``short``: the
        list :meth:`short_form` speaks of (the caller vouches that no row has as many cached slots as the split
        form begins at; the results are those of the default list either way, up to the order of fp32 sums)."""
        stream = torch.cuda.current_stream(self.device).cuda_stream
        short = short and self._table_short is not None
        table, calls = (self._table_short, self._calls_short) if short else (self._table, self._calls)
        with ops._on(self.device):
            rc = _lib.load().vrl_decode_run_calls(table, len(table), ctypes.byref(self._failed_at), stream)
        if rc:
            # a step that stopped half-way may leave the split attention's arrival counters above zero,
            # and every later launch over that workspace would then merge too early: clear them
            if self._split_ws is not None and not torch.cuda.is_current_stream_capturing():
                self._split_ws.zero_()
            _lib.check(rc, calls[self._failed_at.value][0].__name__)
        return self.normed
