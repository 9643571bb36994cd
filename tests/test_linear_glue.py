"""``Int4Linear`` and the policy glue: structure on CPU, numerics on the GPU.

The stand-in policy mirrors the accessors the reference exposes
(``JanusProPolicy._lm_trunk`` / ``_base``, vrl/models/families/janus_pro/policy.py:226-266)
around a real, randomly initialised Hugging Face ``LlamaModel`` built offline from a config,
the way the reference's own tests stub the trunk (tests/models/test_janus_wrapper.py:30-87).
"""

import types

import pytest
import torch
from torch import nn

from visionrl_amd.linear import Int4GateUpSiLU, Int4Linear, Int4LlamaMLP
from visionrl_amd.policy_glue import (apply_int4_to_policy, build_int4_runtime_bundle,
                                      int4_options_from_spec)

HIDDEN, INTER, HEADS, LAYERS, VOCAB_IMG = 256, 512, 4, 2, 1024


def tiny_llama():
    from transformers import LlamaConfig, LlamaModel

    cfg = LlamaConfig(hidden_size=HIDDEN, intermediate_size=INTER, num_hidden_layers=LAYERS,
                      num_attention_heads=HEADS, num_key_value_heads=HEADS, vocab_size=128,
                      max_position_embeddings=64)
    torch.manual_seed(0)
    return LlamaModel(cfg).to(torch.bfloat16).eval()


class StubMMGPT(nn.Module):
    def __init__(self):
        super().__init__()
        self.language_model = types.SimpleNamespace(model=tiny_llama())
        torch.manual_seed(1)
        self.gen_head = nn.Linear(HIDDEN, VOCAB_IMG, bias=False).to(torch.bfloat16)


class StubPolicy:
    """Only the two accessors the glue uses."""

    def __init__(self):
        self.mmgpt = StubMMGPT()

    def _base(self):
        return self.mmgpt

    def _lm_trunk(self):
        return self.mmgpt.language_model.model


def test_apply_swaps_every_decode_linear():
    policy = StubPolicy()
    summary = apply_int4_to_policy(policy, group_size=128)
    # nothing is prepacked on the CPU: the MFMA-shaped copies are made only for weights on a GPU
    assert summary == {"linears": 7 * LAYERS, "fused_mlps": LAYERS, "head_linears": 1, "group_size": 128,
                       "prepacked": 0, "dense_kept": 0, "qkv_groups": 0}
    for layer in policy._lm_trunk().layers:
        for name in ("q_proj", "k_proj", "v_proj", "o_proj"):
            mod = getattr(layer.self_attn, name)
            assert isinstance(mod, Int4Linear)
            assert (mod.in_features, mod.out_features) == (HIDDEN, HIDDEN)
            assert mod.qweight.shape == (HIDDEN, HIDDEN // 8) and mod.qweight.dtype == torch.int32
            assert mod.scales.shape == (HIDDEN, HIDDEN // 128) and mod.scales.dtype == torch.bfloat16
        assert isinstance(layer.mlp, Int4LlamaMLP)
        assert isinstance(layer.mlp.gate_up, Int4GateUpSiLU)
        assert layer.mlp.gate_up.qweight.shape == (2 * INTER, HIDDEN // 8)
        assert layer.mlp.down_proj.in_features == INTER
    assert isinstance(policy._base().gen_head, Int4Linear)
    # nothing left to do on a second pass
    again = apply_int4_to_policy(policy, group_size=128)
    assert again["linears"] == 0 and again["fused_mlps"] == 0 and again["head_linears"] == 0


def test_targets_and_unfused_mlp():
    policy = StubPolicy()
    summary = apply_int4_to_policy(policy, group_size=64, targets=("q_proj", "v_proj", "down_proj"),
                                   fuse_mlp=True, head=False)
    assert summary["linears"] == 3 * LAYERS and summary["fused_mlps"] == 0 and summary["head_linears"] == 0
    layer = policy._lm_trunk().layers[0]
    assert isinstance(layer.self_attn.q_proj, Int4Linear) and layer.self_attn.q_proj.group_size == 64
    assert isinstance(layer.self_attn.k_proj, nn.Linear)
    assert isinstance(layer.mlp.down_proj, Int4Linear) and isinstance(layer.mlp.gate_proj, nn.Linear)
    assert isinstance(policy._base().gen_head, nn.Linear)
    with pytest.raises(ValueError):
        apply_int4_to_policy(policy, targets=("lm_head",))


def test_lora_wrapper_keeps_its_adapter():
    """A PEFT-style wrapper (frozen weight in ``base_layer``) gets only its base quantised."""

    class LoraLike(nn.Module):
        def __init__(self, base):
            super().__init__()
            self.base_layer = base
            self.lora_A = nn.Linear(base.in_features, 4, bias=False)
            self.lora_B = nn.Linear(4, base.out_features, bias=False)

        def forward(self, x):
            return self.base_layer(x) + self.lora_B(self.lora_A(x))

    policy = StubPolicy()
    attn = policy._lm_trunk().layers[0].self_attn
    attn.q_proj = LoraLike(attn.q_proj)
    apply_int4_to_policy(policy, head=False)
    assert isinstance(attn.q_proj, LoraLike)
    assert isinstance(attn.q_proj.base_layer, Int4Linear)
    assert isinstance(attn.q_proj.lora_A, nn.Linear)


def test_lora_only_weight_sync_leaves_the_int4_base_alone():
    """The rollout worker's update path (worker.py:55-71) on an int4 policy: adapter tensors are copied
    in place, base weights of the trainer's state dict are skipped, misfits are refused."""
    from visionrl_amd.policy_glue import install_lora_weight_sync

    class LoraLike(nn.Module):
        def __init__(self, base):
            super().__init__()
            self.base_layer = base
            self.lora_A = nn.ModuleDict({"default": nn.Linear(base.in_features, 4, bias=False)})
            self.lora_B = nn.ModuleDict({"default": nn.Linear(4, base.out_features, bias=False)})

        def forward(self, x):
            return self.base_layer(x) + self.lora_B["default"](self.lora_A["default"](x))

    class ModulePolicy(nn.Module):       # the reference's policy is an nn.Module holding the network
        def __init__(self):
            super().__init__()
            self.trunk = tiny_llama()
            for layer in self.trunk.layers:
                layer.self_attn.q_proj = LoraLike(layer.self_attn.q_proj)

        def _lm_trunk(self):
            return self.trunk

    trainer, rollout = ModulePolicy(), ModulePolicy()
    apply_int4_to_policy(rollout, group_size=128, head=False)
    install_lora_weight_sync(rollout)
    state = trainer.state_dict()                             # what the trainer exports: everything
    for key in state:
        if "lora_" in key:
            state[key] = torch.randn_like(state[key])
    before = {k: v.clone() for k, v in rollout.state_dict().items()}
    ptrs = {k: v.data_ptr() for k, v in rollout.state_dict().items()}
    summary = rollout.load_trainable_state(state)
    assert summary["loaded"] == 2 * LAYERS and summary["skipped"] == len(state) - 2 * LAYERS
    after = rollout.state_dict()
    for key, value in after.items():
        assert value.data_ptr() == ptrs[key]                  # in place: plans and graphs stay valid
        if "lora_" in key:
            assert torch.equal(value, state[key].to(value.dtype))
        else:
            assert torch.equal(value, before[key])            # qweight / scales / qzeros untouched
    with pytest.raises(ValueError, match="no adapter"):
        rollout.load_trainable_state({k: v for k, v in state.items() if "lora_" not in k})
    bad = {k: (v[:1] if "lora_A" in k else v) for k, v in state.items()}
    with pytest.raises(ValueError, match="shape"):
        rollout.load_trainable_state(bad)
    with pytest.raises(ValueError, match="no such adapter"):
        rollout.load_trainable_state({"trunk.layers.9.self_attn.q_proj.lora_A.default.weight":
                                      torch.zeros(4, HIDDEN)})


def test_state_dict_round_trip():
    lin = nn.Linear(256, 48, bias=True).to(torch.bfloat16)
    a = Int4Linear.from_linear(lin, 64)
    b = Int4Linear(256, 48, 64, bias=True)
    b.load_state_dict(a.state_dict())
    for k, v in a.state_dict().items():
        assert torch.equal(v, b.state_dict()[k]), k
    assert set(a.state_dict()) == {"qweight", "scales", "qzeros", "bias"}
    with pytest.raises(ValueError):
        Int4Linear(250, 48, 128)


def test_runtime_spec_options_and_builder_wrapper():
    spec = types.SimpleNamespace(extra={})
    assert int4_options_from_spec(spec) is None
    spec.extra["int4"] = True
    assert int4_options_from_spec(spec)["group_size"] == 128
    spec.extra["int4"] = {"group_size": 64, "head": False}
    opt = int4_options_from_spec(spec)
    assert opt["group_size"] == 64 and opt["head"] is False and opt["fuse_mlp"] is True
    spec.extra["int4"] = {"bits": 3}
    with pytest.raises(ValueError):
        int4_options_from_spec(spec)
    spec.extra["int4"] = "yes"
    with pytest.raises(TypeError):
        int4_options_from_spec(spec)

    spec.extra["int4"] = {"group_size": 128}
    bundle = build_int4_runtime_bundle(
        spec, lambda s: types.SimpleNamespace(policy=StubPolicy(), metadata={"model_path": "stub"}))
    assert bundle.metadata["int4"]["linears"] == 7 * LAYERS
    assert isinstance(bundle.policy._base().gen_head, Int4Linear)
    assert bundle.metadata["int4"]["static_sampler"] is False    # this stand-in has no sample_image_tokens to replace

    class Sampling(StubPolicy):                                   # a policy with the loop and what the loop needs
        def __init__(self):
            super().__init__()
            self.mmgpt.prepare_gen_img_embeds = lambda ids: None

        def sample_image_tokens(self, *args, **kwargs):
            raise AssertionError("replaced by the static sampler")

    for wanted in (True, False):
        spec.extra["int4"] = {"static_sampler": wanted}
        b = build_int4_runtime_bundle(spec, lambda s: types.SimpleNamespace(policy=Sampling(), metadata={}))
        assert b.metadata["int4"]["static_sampler"] is wanted
        assert hasattr(b.policy, "_static_ar_sampler") is wanted
        assert (b.policy.sample_image_tokens.__func__ is not Sampling.sample_image_tokens) is wanted
    plain = build_int4_runtime_bundle(types.SimpleNamespace(extra={}),
                                      lambda s: types.SimpleNamespace(policy=StubPolicy(), metadata={}))
    assert "int4" not in plain.metadata
    assert isinstance(plain.policy._base().gen_head, nn.Linear)


def test_cpu_forward_fails_loudly():
    lin = Int4Linear.from_linear(nn.Linear(128, 8, bias=False).to(torch.bfloat16), 128)
    with pytest.raises(ValueError, match="no CPU path"):
        lin(torch.zeros(1, 128, dtype=torch.bfloat16))
    with pytest.raises(TypeError):
        lin(torch.zeros(1, 128, dtype=torch.float32))


# ---------------------------------------------------------------------- GPU numerics
@pytest.mark.gpu
def test_int4_linear_matches_dequantised_linear():
    dev = "cuda:0"
    torch.manual_seed(2)
    lin = nn.Linear(512, 96, bias=True).to(torch.bfloat16).to(dev)
    q = Int4Linear.from_linear(lin, 128)
    x = torch.randn(3, 5, 512, device=dev).to(torch.bfloat16)
    w = q.dequantize()
    assert w.shape == (96, 512) and w.dtype == torch.bfloat16
    ref = (x.reshape(-1, 512).double() @ w.double().t()).reshape(3, 5, 96)
    y = q(x)
    assert y.shape == (3, 5, 96) and y.dtype == torch.bfloat16
    err = (y.double() - (ref + q.bias.double())).abs()
    assert (err <= 2.0 ** -7 * ref.abs() + 2.0 ** -6).all()
    # the quantiser keeps the weights within one step
    step = q.scales.float().repeat_interleave(128, dim=1)
    assert ((w.float() - lin.weight.float()).abs() <= 1.01 * step).all()


@pytest.mark.gpu
def test_swapped_trunk_tracks_the_dequantised_trunk():
    """int4 modules vs the same model running nn.Linear on the dequantised weights: one decode
    step with a KV cache, as the reference drives the trunk (policy.py:673-678)."""
    dev = "cuda:0"
    policy = StubPolicy()
    policy.mmgpt.to(dev)
    policy.mmgpt.language_model.model.to(dev)
    reference = StubPolicy()
    reference.mmgpt.to(dev)
    reference.mmgpt.language_model.model.to(dev)
    reference._lm_trunk().load_state_dict(policy._lm_trunk().state_dict())
    reference.mmgpt.gen_head.load_state_dict(policy.mmgpt.gen_head.state_dict())

    summary = apply_int4_to_policy(policy, group_size=128)
    # every quantised module got its prepacked copy: q/k/v/o + gate||up + down per layer, and the head
    assert summary["prepacked"] == 6 * LAYERS + 1
    assert summary["qkv_groups"] == LAYERS       # q|k|v of every layer share one launch per decode step
    # give the reference copy the dequantised weights
    for lq, lr in zip(policy._lm_trunk().layers, reference._lm_trunk().layers):
        for name in ("q_proj", "k_proj", "v_proj", "o_proj"):
            getattr(lr.self_attn, name).weight.data.copy_(getattr(lq.self_attn, name).dequantize())
        gu = lq.mlp.gate_up
        from visionrl_amd import ops
        w = ops.int4_dequant(gu.qweight, gu.scales, gu.qzeros, gu.group_size)
        lr.mlp.gate_proj.weight.data.copy_(w[:INTER])
        lr.mlp.up_proj.weight.data.copy_(w[INTER:])
        lr.mlp.down_proj.weight.data.copy_(lq.mlp.down_proj.dequantize())
    reference.mmgpt.gen_head.weight.data.copy_(policy.mmgpt.gen_head.dequantize())

    torch.manual_seed(3)
    prompt = torch.randn(2, 6, HIDDEN, device=dev).to(torch.bfloat16) * 0.5
    step = torch.randn(2, 1, HIDDEN, device=dev).to(torch.bfloat16) * 0.5
    outs = []
    with torch.no_grad():
        for pol in (policy, reference):
            trunk = pol._lm_trunk()
            pre = trunk(inputs_embeds=prompt, use_cache=True)
            dec = trunk(inputs_embeds=step, past_key_values=pre.past_key_values, use_cache=True)
            logits = pol._base().gen_head(dec.last_hidden_state[:, -1:, :])
            outs.append((pre.last_hidden_state.float(), dec.last_hidden_state.float(), logits.float()))
    for a, b in zip(outs[0], outs[1]):
        assert a.shape == b.shape
        assert torch.isfinite(a).all()
        # same weights, bf16 activations everywhere: only accumulation order and the fused
        # fp32 SiLU epilogue differ
        assert (a - b).abs().max() <= 0.05 * b.abs().max() + 1e-3
    assert outs[0][2].shape == (2, 1, VOCAB_IMG)


@pytest.mark.gpu
def test_prepacked_module_path_agrees_with_the_canonical_one():
    """Decode-sized calls go through the plan-free launch once a module is prepacked; larger ones
    keep the canonical kernels.  Both are the same arithmetic up to fp32 summation order."""
    dev = "cuda:0"
    torch.manual_seed(4)
    lin = nn.Linear(1024, 160, bias=False).to(torch.bfloat16).to(dev)
    q = Int4Linear.from_linear(lin, 128)
    w = q.dequantize().double()
    for rows in (1, 5, 16, 40):
        x = torch.randn(rows, 1024, device=dev).to(torch.bfloat16)
        plain = q(x)
        q.prepack_()
        assert q._packed is not None and q._direct_rows == 32
        fast = q(x)
        del q._packed
        ref = x.double() @ w.t()
        for y in (plain, fast):
            assert (y.double() - ref).abs().le(2.0 ** -7 * ref.abs() + 2.0 ** -6).all()
        if rows > 16:
            assert torch.equal(plain, fast)      # same kernel: beyond 16 rows the prepacked copy is not used


@pytest.mark.gpu
def test_grouped_siblings_hand_results_over_by_tensor_identity():
    """q|k|v grouped: the leader's launch computes all three; a sibling returns the handed result only
    for the very same input object, and computes on its own otherwise."""
    dev = "cuda:0"
    torch.manual_seed(6)
    mods = [Int4Linear.from_linear(nn.Linear(512, n, bias=(n == 96)).to(torch.bfloat16).to(dev), 128).prepack_()
            for n in (128, 96, 64)]
    alone = [Int4Linear.from_packed(m.qweight, m.scales, m.qzeros, 128, bias=m.bias).prepack_() for m in mods]
    q, k, v = mods
    q.group_with(k, v)
    x = torch.randn(2, 1, 512, device=dev).to(torch.bfloat16)
    want = [m(x) for m in alone]
    got_q = q(x)
    assert k._handed is not None and v._handed is not None
    got_k, got_v = k(x), v(x)
    assert k._handed is None and v._handed is None
    for a, b in zip(want, (got_q, got_k, got_v)):
        assert torch.equal(a, b)                         # same kernel body, one tile per workgroup either way
    # another tensor with equal contents is not the same input: the sibling computes it itself
    q(x)
    other = x.clone() * 2
    assert torch.equal(k(other), alone[1](other))
    assert torch.equal(v(x), want[2])                    # v still takes what q handed it for x
    # more rows than the plan-free launch takes: every module on its own
    big = torch.randn(40, 512, device=dev).to(torch.bfloat16)
    assert torch.equal(q(big), alone[0](big)) and k._handed is None


@pytest.mark.gpu
def test_prompt_sized_calls_go_through_the_library_gemm():
    """More than 32 rows (the prompt pass): bit-exact weight tile, then the library GEMM, for the plain
    and the fused gate|up module, prepacked or not."""
    import torch.nn.functional as F

    dev = "cuda:0"
    torch.manual_seed(4)
    lin = nn.Linear(512, 96, bias=False).to(torch.bfloat16).to(dev)
    gate = nn.Linear(512, 64, bias=False).to(torch.bfloat16).to(dev)
    up = nn.Linear(512, 64, bias=False).to(torch.bfloat16).to(dev)
    x = torch.randn(4, 20, 512, device=dev).to(torch.bfloat16)   # 80 rows
    q = Int4Linear.from_linear(lin, 128)
    gu = Int4GateUpSiLU(Int4Linear.from_linear(gate, 128), Int4Linear.from_linear(up, 128))
    for prepacked in (False, True):
        if prepacked:
            q.prepack_(), gu.prepack_()
            assert q._packed is not None and gu._packed is not None
        y = q(x)
        assert torch.equal(y, F.linear(x, q.dequantize()))
        from visionrl_amd import ops

        w = ops.int4_dequant(gu.qweight, gu.scales, gu.qzeros, 128)
        g, u = F.linear(x, w).chunk(2, dim=-1)
        got = gu(x)
        assert got.shape == (4, 20, 64) and torch.equal(got, F.silu(g) * u)
        # and it stays within a bf16 rounding or two of the fused decode kernel's fp32 epilogue
        small = gu(x[:1, :8])
        assert (small.float() - got[:1, :8].float()).abs().max().item() <= 2.0 ** -6 * max(1.0, got.abs().max().item())


@pytest.mark.gpu
def test_kept_dense_weight_serves_prompt_sized_calls_until_the_source_changes():
    """``keep_dense_()``: prompt-sized and gradient-carrying calls multiply by one kept bf16 tensor (the
    same results, no dequantisation per call); a write to the canonical buffers makes the next call
    rebuild it; ``keep_dense_(False)`` drops it."""
    import torch.nn.functional as F

    dev = "cuda:0"
    torch.manual_seed(14)
    q = Int4Linear.from_linear(nn.Linear(512, 96, bias=False).to(torch.bfloat16).to(dev), 128).prepack_()
    gu = Int4GateUpSiLU(Int4Linear.from_linear(nn.Linear(512, 64, bias=False).to(torch.bfloat16).to(dev), 128),
                        Int4Linear.from_linear(nn.Linear(512, 64, bias=False).to(torch.bfloat16).to(dev), 128)).prepack_()
    x = torch.randn(80, 512, device=dev).to(torch.bfloat16)
    want_q, want_gu = q(x), gu(x)
    q.keep_dense_(), gu.keep_dense_()
    assert torch.equal(q(x), want_q) and torch.equal(gu(x), want_gu)
    kept = q._dense[1]
    assert torch.equal(kept, q.dequantize())
    assert torch.equal(q(x), want_q) and q._dense[1] is kept          # the second call reuses the tensor
    xg = x.clone().requires_grad_(True)
    q(xg).float().sum().backward()                                     # and so does the replay's route
    assert q._dense[1] is kept and xg.grad is not None
    small = x[:2]
    assert torch.equal(q(small), Int4Linear.from_packed(q.qweight, q.scales, q.qzeros, 128).prepack_()(small))
    # a new weight: the kept tensor and the prepacked copy are both rebuilt on the next call
    other = Int4Linear.from_linear(nn.Linear(512, 96, bias=False).to(torch.bfloat16).to(dev), 128)
    q.load_state_dict(other.state_dict())
    assert torch.equal(q(x), F.linear(x, other.dequantize())) and q._dense[1] is not kept
    q.keep_dense_(False)
    assert q._dense is None and torch.equal(q(x), F.linear(x, other.dequantize())) and q._dense is None


def test_keep_dense_option_reaches_every_quantised_module():
    from visionrl_amd.policy_glue import apply_int4_to_policy, int4_options_from_spec

    policy = StubPolicy()
    summary = apply_int4_to_policy(policy, prepack=False, keep_dense=True)
    assert summary["dense_kept"] == 6 * LAYERS + 1      # q, k, v, o, gate|up, down per layer, and the head
    kinds = (Int4Linear, Int4GateUpSiLU)
    assert all(getattr(m, "_keep_dense", False) for m in policy.mmgpt.modules() if isinstance(m, kinds))

    class Spec:
        extra = {"int4": {"keep_dense": True}}
    assert int4_options_from_spec(Spec())["keep_dense"] is True


@pytest.mark.gpu
def test_gradient_reaches_the_input_of_a_quantised_layer():
    """A train-time replay over the frozen int4 base (inputs that carry a gradient, any row count): the
    modules multiply by the dequantised weight through autograd-recorded ops, so ``x.grad`` is that of
    the explicit bf16 product; without a gradient the same decode-sized call takes the HIP launch."""
    import torch.nn.functional as F

    dev = "cuda:0"
    torch.manual_seed(5)
    q = Int4Linear.from_linear(nn.Linear(512, 96, bias=True).to(torch.bfloat16).to(dev), 128).prepack_()
    gu = Int4GateUpSiLU(Int4Linear.from_linear(nn.Linear(512, 64, bias=False).to(torch.bfloat16).to(dev), 128),
                        Int4Linear.from_linear(nn.Linear(512, 64, bias=False).to(torch.bfloat16).to(dev), 128)).prepack_()
    for rows in (2, 48):
        x = torch.randn(rows, 512, device=dev).to(torch.bfloat16).requires_grad_(True)
        ref = x.detach().clone().requires_grad_(True)
        y = q(x)
        assert y.requires_grad
        y.float().square().sum().backward()
        (F.linear(ref, q.dequantize()) + q.bias).float().square().sum().backward()
        assert torch.equal(x.grad, ref.grad)
        x.grad = ref.grad = None
        z = gu(x)
        assert z.requires_grad
        z.float().sum().backward()
        from visionrl_amd import ops
        g, u = F.linear(ref, ops.int4_dequant(gu.qweight, gu.scales, gu.qzeros, 128)).chunk(2, dim=-1)
        (F.silu(g) * u).float().sum().backward()
        assert torch.equal(x.grad, ref.grad)
        with torch.no_grad():
            assert not q(x).requires_grad and not gu(x).requires_grad


def test_a_prepacked_copy_knows_when_its_source_changed():
    """The canonical buffers are the module's state; the prepacked copy is derived from them and is
    stale after an in-place write (``load_state_dict``) or a replaced buffer (``.to()``).  Where torch keeps
    no modification counter for a buffer (an inference tensor) the copy is tied to the tensor object, its
    address and shape: such a module does not repack on every call, and ``prepack_()`` follows an edit."""
    from visionrl_amd.linear import _source_changed, _source_state

    a, b = torch.zeros(4), torch.ones(4)
    state = _source_state(a, b)
    assert not _source_changed(state, a, b)
    b.add_(1)
    assert _source_changed(state, a, b)
    state = _source_state(a, b)
    assert _source_changed(state, a.clone(), b)
    with torch.inference_mode():
        c = torch.zeros(4)
        d = torch.zeros(4)
    state = _source_state(c)
    assert not _source_changed(state, c)        # the same object in the same place: not stale
    assert _source_changed(state, d)            # another tensor
    del d
    state = _source_state(a)
    del a                                       # the source is gone: whatever stands in its place is new
    assert _source_changed(state, torch.zeros(4))
    mod = Int4Linear(128, 16, 128)
    assert not mod.packed_is_stale()                 # nothing prepacked
    mod._packed, mod._packed_from = object(), _source_state(mod.qweight, mod.scales, mod.qzeros)
    assert not mod.packed_is_stale()
    mod.load_state_dict({k: v.clone() + 1 for k, v in mod.state_dict().items()})
    assert mod.packed_is_stale()
    assert mod._fresh_packed() is None               # made again: on the CPU there is no prepacked form


@pytest.mark.gpu
def test_hand_over_is_void_once_the_input_was_written_or_the_leader_ran_again():
    """A persistent input buffer rewritten in place between q_proj(x) and k_proj(x), and a k_proj call
    that follows a step in which it was skipped: the sibling computes from what x holds now."""
    dev = "cuda:0"
    torch.manual_seed(8)
    mods = [Int4Linear.from_linear(nn.Linear(512, n, bias=False).to(torch.bfloat16).to(dev), 128).prepack_()
            for n in (128, 96, 64)]
    alone = [Int4Linear.from_packed(m.qweight, m.scales, m.qzeros, 128).prepack_() for m in mods]
    q, k, v = mods
    q.group_with(k, v)
    x = torch.randn(2, 1, 512, device=dev).to(torch.bfloat16)
    first = [m(x) for m in alone]
    q(x)
    assert k._handed is not None
    x.mul_(-3)                                           # the same tensor object, other contents
    now = [m(x) for m in alone]
    assert torch.equal(k(x), now[1]) and not torch.equal(now[1], first[1])
    assert torch.equal(v(x), now[2])
    # step 1 hands over, k is skipped; step 2 reuses the buffer: the leader's new call voids the old results
    q(x)
    x.copy_(torch.randn_like(x))
    assert torch.equal(q(x), alone[0](x)) and torch.equal(k(x), alone[1](x)) and torch.equal(v(x), alone[2](x))
    # a leader call that takes another route (too many rows for the grouped launch) leaves nothing behind
    q(x)
    big = torch.randn(40, 512, device=dev).to(torch.bfloat16)
    q(big)
    assert k._handed is None and v._handed is None
    # inputs without a modification counter are never handed over
    with torch.inference_mode():
        xi = torch.randn(2, 512, device=dev).to(torch.bfloat16)
        yq = q(xi)
        assert k._handed is None and torch.equal(yq, alone[0](xi)) and torch.equal(k(xi), alone[1](xi))


@pytest.mark.gpu
def test_loading_a_state_dict_into_a_prepacked_module_refreshes_the_decode_path():
    """Decode-sized calls stream the prepacked copy, prompt-sized ones and dequantize() the canonical
    buffers: after ``load_state_dict`` both must follow the new weights."""
    dev = "cuda:0"
    torch.manual_seed(9)
    old = Int4Linear.from_linear(nn.Linear(512, 96, bias=False).to(torch.bfloat16).to(dev), 128).prepack_()
    new = Int4Linear.from_linear(nn.Linear(512, 96, bias=False).to(torch.bfloat16).to(dev), 128).prepack_()
    x = torch.randn(3, 512, device=dev).to(torch.bfloat16)
    before, want = old(x), new(x)
    assert not torch.equal(before, want)
    blob = old._packed
    old.load_state_dict(new.state_dict())
    assert old.packed_is_stale()
    assert torch.equal(old(x), want) and old._packed is not blob and not old.packed_is_stale()
    gu_old = Int4GateUpSiLU(Int4Linear.from_linear(nn.Linear(512, 64, bias=False).to(torch.bfloat16).to(dev), 128),
                            Int4Linear.from_linear(nn.Linear(512, 64, bias=False).to(torch.bfloat16).to(dev), 128)).prepack_()
    gu_new = Int4GateUpSiLU(Int4Linear.from_linear(nn.Linear(512, 64, bias=False).to(torch.bfloat16).to(dev), 128),
                            Int4Linear.from_linear(nn.Linear(512, 64, bias=False).to(torch.bfloat16).to(dev), 128)).prepack_()
    want = gu_new(x)
    gu_old.load_state_dict(gu_new.state_dict())
    assert torch.equal(gu_old(x), want)
    # a grouped leader notices a stale sibling and a refreshed sibling rebuilds the group's launch
    q = Int4Linear.from_linear(nn.Linear(512, 128, bias=False).to(torch.bfloat16).to(dev), 128).prepack_()
    q.group_with(old)
    old.load_state_dict(Int4Linear.from_linear(nn.Linear(512, 96, bias=False).to(torch.bfloat16).to(dev), 128).state_dict())
    fresh = Int4Linear.from_packed(old.qweight, old.scales, old.qzeros, 128).prepack_()
    x3 = x.reshape(1, 3, 512)
    q(x3)
    assert old._handed is None                           # the sibling's copy was stale: no hand-over
    assert torch.equal(old(x3), fresh(x3))
    q(x3)
    assert old._handed is not None and torch.equal(old(x3), fresh(x3))
