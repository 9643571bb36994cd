"""Loader glue: swap a Janus-Pro style policy's decode linears for int4 modules.

Hook points in the reference (all under ``vrl/models/families/janus_pro/``):

* ``policy.py:240-266``  ``JanusProPolicy._lm_trunk()`` returns the Hugging Face
  ``LlamaModel`` whose ``layers[i].self_attn.{q,k,v,o}_proj`` and
  ``layers[i].mlp.{gate,up,down}_proj`` are ``nn.Linear``.
* ``policy.py:226-238``, ``:138-160``  ``_base().gen_head`` maps hidden states to
  image-token logits.
* ``policy.py:298-324``  LoRA: PEFT wraps target linears; the wrapper keeps the
  frozen weight in ``base_layer`` and adds ``scaling * B(A(x))``.  Only
  ``base_layer`` is replaced, so the adapter keeps working on top of int4.
* ``builder.py:11-33``, ``:77-113`` and ``vrl/distributed/ray/rollout/worker.py:143-163``:
  rollout workers build the policy from a ``RuntimeBuildSpec`` whose ``extra``
  dict is the only channel for new scalar options; ``extra["int4"]`` carries
  ``{"group_size": 128, "targets": [...], "fuse_mlp": true, "head": true, "prepack": true, "group_qkv": true, "keep_dense": false,
  "static_sampler": true}`` (the last one routes ``sample_image_tokens`` and the step API through
  :mod:`visionrl_amd.ar_decode`).

* ``vrl/distributed/ray/rollout/worker.py:55-71``: a rollout worker applies synced trainer
  weights through ``policy.load_trainable_state(state)``, which the Janus-Pro policy does not
  define (the diffusion policies do, ``vrl/models/diffusion.py:233-256``);
  :func:`install_lora_weight_sync` gives an int4 policy that method for the
  ``sync_trainable_state: "lora_only"`` mode (``vrl/rollouts/runtime/config.py:20-37``).

Nothing here imports the reference; the policy is duck-typed.
"""

from __future__ import annotations

import types
from typing import Any, Callable, Iterable, Mapping

import torch
from torch import nn

from .linear import Int4GateUpSiLU, Int4Linear, Int4LlamaMLP

ATTN_TARGETS = ("q_proj", "k_proj", "v_proj", "o_proj")
MLP_TARGETS = ("gate_proj", "up_proj", "down_proj")
DEFAULT_TARGETS = ATTN_TARGETS + MLP_TARGETS


def _trunk(policy: Any) -> nn.Module:
    if hasattr(policy, "_lm_trunk"):
        return policy._lm_trunk()
    if isinstance(policy, nn.Module) and hasattr(policy, "layers"):
        return policy
    raise TypeError("expected a policy exposing _lm_trunk() or a LlamaModel-like trunk with .layers")


def _head_owner(policy: Any):
    base = policy._base() if hasattr(policy, "_base") else policy
    return base if hasattr(base, "gen_head") else None


def _quantizable(linear: nn.Module, group_size: int) -> bool:
    return isinstance(linear, nn.Linear) and linear.in_features % group_size == 0


def _swap_linear(parent: nn.Module, name: str, group_size: int) -> bool:
    """Replace ``parent.name`` (or its PEFT ``base_layer``) by an ``Int4Linear``."""
    child = getattr(parent, name, None)
    if child is None:
        return False
    if isinstance(child, Int4Linear):
        return False
    inner = getattr(child, "base_layer", None)
    if inner is not None and not isinstance(child, nn.Linear):
        # PEFT LoRA wrapper: keep the adapter, quantise the frozen base weight
        if _quantizable(inner, group_size):
            child.base_layer = Int4Linear.from_linear(inner, group_size)
            return True
        return False
    if _quantizable(child, group_size):
        setattr(parent, name, Int4Linear.from_linear(child, group_size))
        return True
    return False


def _int4_of(module):
    """The ``Int4Linear`` behind ``module``: itself, or the ``base_layer`` of a PEFT wrapper."""
    if isinstance(module, Int4Linear):
        return module
    inner = getattr(module, "base_layer", None)
    return inner if isinstance(inner, Int4Linear) else None


def _swap_all_linears(module: nn.Module, group_size: int) -> int:
    n = 0
    for name, child in list(module.named_children()):
        if isinstance(child, nn.Linear):
            n += int(_swap_linear(module, name, group_size))
        else:
            n += _swap_all_linears(child, group_size)
    return n


def apply_int4_to_policy(policy: Any, group_size: int = 128,
                         targets: Iterable[str] = DEFAULT_TARGETS, fuse_mlp: bool = True,
                         head: bool = True, prepack: bool = True, group_qkv: bool = True,
                         keep_dense: bool = False) -> dict:
    """Quantise the decode linears of ``policy`` in place; returns a count summary.

    ``fuse_mlp`` replaces a whole MLP block by :class:`Int4LlamaMLP` (gate||up with
    the SiLU epilogue in one launch) when all three projections are targeted and
    none of them carries a LoRA adapter.  ``prepack`` keeps a second, MFMA-shaped copy
    of every quantised weight that lives on a GPU, which decode-sized calls (up to 32
    activation rows) stream through the plan-free launch; with ``group_qkv`` the three
    projections of an attention block then share one launch per decode step.
    ``keep_dense`` also keeps the dequantised bf16 weight of every quantised module (four times
    the int4 bytes) so that prompt passes and the train-time replay's micro-batches stop rebuilding
    it on every call.
    """
    targets = tuple(targets)
    unknown = set(targets) - set(DEFAULT_TARGETS)
    if unknown:
        raise ValueError(f"unknown int4 targets {sorted(unknown)}; choose from {DEFAULT_TARGETS}")
    trunk = _trunk(policy)
    summary = {"linears": 0, "fused_mlps": 0, "head_linears": 0, "group_size": int(group_size)}
    for layer in trunk.layers:
        attn, mlp = getattr(layer, "self_attn", None), getattr(layer, "mlp", None)
        if attn is not None:
            for name in ATTN_TARGETS:
                if name in targets:
                    summary["linears"] += int(_swap_linear(attn, name, group_size))
        if mlp is None:
            continue
        wants_all = all(n in targets for n in MLP_TARGETS)
        plain = all(isinstance(getattr(mlp, n, None), nn.Linear) and
                    _quantizable(getattr(mlp, n), group_size) and getattr(mlp, n).bias is None
                    for n in MLP_TARGETS)
        if fuse_mlp and wants_all and plain:
            layer.mlp = Int4LlamaMLP(mlp, group_size)
            summary["fused_mlps"] += 1
            summary["linears"] += 3
        else:
            for name in MLP_TARGETS:
                if name in targets:
                    summary["linears"] += int(_swap_linear(mlp, name, group_size))
    owner = _head_owner(policy)
    if head and owner is not None:
        if isinstance(owner.gen_head, nn.Linear):
            summary["head_linears"] += int(_swap_linear(owner, "gen_head", group_size))
        else:
            summary["head_linears"] += _swap_all_linears(owner.gen_head, group_size)
    summary["prepacked"] = 0
    if prepack:
        roots = [trunk] + ([owner.gen_head] if head and owner is not None else [])
        for root in roots:
            for mod in root.modules():
                if isinstance(mod, (Int4Linear, Int4GateUpSiLU)):
                    mod.prepack_()
                    summary["prepacked"] += int(getattr(mod, "_packed", None) is not None)
    summary["dense_kept"] = 0
    if keep_dense:
        roots = [trunk] + ([owner.gen_head] if head and owner is not None else [])
        for root in roots:
            for mod in root.modules():
                if isinstance(mod, (Int4Linear, Int4GateUpSiLU)):
                    mod.keep_dense_()
                    summary["dense_kept"] += 1
    summary["qkv_groups"] = 0
    if prepack and group_qkv:
        for layer in trunk.layers:
            attn = getattr(layer, "self_attn", None)
            members = [_int4_of(getattr(attn, n, None)) for n in ("q_proj", "k_proj", "v_proj")] if attn else []
            if members and all(m is not None and getattr(m, "_packed", None) is not None for m in members):
                members[0].group_with(*members[1:])
                summary["qkv_groups"] += 1
    return summary


def int4_options_from_spec(spec: Any) -> dict | None:
    """Read ``spec.extra["int4"]``; ``None`` when int4 is not requested.

    Accepts ``True`` (defaults) or a dict of scalars/lists, the only kinds of
    value the reference lets cross its process boundary.
    """
    extra = getattr(spec, "extra", None) or {}
    opt = extra.get("int4")
    if opt is None or opt is False:
        return None
    if opt is True:
        opt = {}
    if not isinstance(opt, dict):
        raise TypeError('RuntimeBuildSpec.extra["int4"] must be true or a dict of options')
    allowed = {"group_size", "targets", "fuse_mlp", "head", "prepack", "group_qkv", "keep_dense", "static_sampler"}
    unknown = set(opt) - allowed
    if unknown:
        raise ValueError(f'unknown keys in extra["int4"]: {sorted(unknown)}')
    return {"group_size": int(opt.get("group_size", 128)),
            "targets": tuple(opt.get("targets", DEFAULT_TARGETS)),
            "fuse_mlp": bool(opt.get("fuse_mlp", True)),
            "head": bool(opt.get("head", True)),
            "prepack": bool(opt.get("prepack", True)),
            "group_qkv": bool(opt.get("group_qkv", True)),
            "keep_dense": bool(opt.get("keep_dense", False)),
            "static_sampler": bool(opt.get("static_sampler", True))}


def build_int4_runtime_bundle(spec: Any, builder: Callable[[Any], Any]) -> Any:
    """Wrap a family runtime builder (``build_janus_pro_runtime_bundle``-shaped).

    Runs ``builder(spec)``, then quantises ``bundle.policy`` if the spec asks for
    it, and records what was done in ``bundle.metadata["int4"]``.
    """
    bundle = builder(spec)
    opt = int4_options_from_spec(spec)
    if opt is not None:
        static_sampler = opt.pop("static_sampler")
        summary = apply_int4_to_policy(bundle.policy, **opt)
        summary["static_sampler"] = False
        if static_sampler and hasattr(bundle.policy, "sample_image_tokens"):
            from .ar_decode import install_static_ar_sampler

            try:   # the image-token loop over a static cache and recorded decode steps
                install_static_ar_sampler(bundle.policy)
                summary["static_sampler"] = True
            except (TypeError, AttributeError):   # not a Janus-Pro shaped policy: leave its own loop
                pass
        meta = getattr(bundle, "metadata", None)
        if isinstance(meta, dict):
            meta["int4"] = summary
    return bundle


# ---------------------------------------------------------------------- weight sync (LoRA only)
def _policy_root(policy: Any) -> nn.Module:
    """The module whose ``state_dict`` keys the trainer's copy of the policy uses."""
    if isinstance(policy, nn.Module):
        return policy
    for name in ("mmgpt", "model"):
        root = getattr(policy, name, None)
        if isinstance(root, nn.Module):
            return root
    raise TypeError("expected an nn.Module policy or one holding its network in .mmgpt / .model")


def load_lora_state(policy: Any, state_dict: Mapping[str, Any], prefix: str = "") -> dict:
    """Copy the adapter tensors of ``state_dict`` into ``policy``; the int4 base stays as it is.

    ``state_dict`` is what the trainer exports for the policy
    (``vrl/trainers/checkpointing.py:217-227``: a full ``state_dict()``) or just its adapter
    part.  Keys with ``lora_`` in them must name a tensor of the same shape in the rollout
    policy and are copied in place (no re-quantisation, no reallocation: captured HIP graphs
    and grouped plans stay valid).  Every other key is a frozen base weight the rollout copy
    holds in int4 and is skipped.  Returns ``{"loaded": n, "skipped": m}``; raises
    ``ValueError`` if there is nothing to load or an adapter key does not fit.
    """
    root = _policy_root(policy)
    own = dict(root.named_parameters())
    own.update(dict(root.named_buffers()))
    loaded = skipped = 0
    problems = []
    with torch.no_grad():
        for key, value in state_dict.items():
            name = key[len(prefix):] if prefix and key.startswith(prefix) else key
            if "lora_" not in name:
                skipped += 1
                continue
            target = own.get(name)
            if target is None:
                problems.append(f"{key}: no such adapter tensor in the rollout policy")
            elif tuple(target.shape) != tuple(value.shape):
                problems.append(f"{key}: shape {tuple(value.shape)} != {tuple(target.shape)}")
            else:
                target.copy_(value.to(device=target.device, dtype=target.dtype))
                loaded += 1
    if problems:
        raise ValueError("adapter state does not fit the rollout policy: " + "; ".join(problems[:5]))
    if loaded == 0:
        raise ValueError("load_trainable_state received no adapter (lora_*) tensors")
    return {"loaded": loaded, "skipped": skipped}


def install_lora_weight_sync(policy: Any, prefix: str = "") -> Any:
    """Give ``policy`` the ``load_trainable_state(state)`` method rollout workers call."""

    def load_trainable_state(self, state_dict: Mapping[str, Any]) -> dict:
        return load_lora_state(self, state_dict, prefix=prefix)

    policy.load_trainable_state = types.MethodType(load_trainable_state, policy)
    return policy
