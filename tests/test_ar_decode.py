"""Static-cache / HIP-graph image-token sampling against the reference's decode loop.

``reference_loop`` restates ``JanusProPolicy.sample_image_tokens`` + ``_sample_ar_step``
(vrl/models/families/janus_pro/policy.py:476-525, :624-731) with plain torch and the trunk's own
dynamic cache: concatenate the rows' caches, call the trunk on ``[cond; uncond]``, head, CFG
combine, softmax -> multinomial, log_softmax -> gather, embed the sampled token for both halves,
append a one to both masks.  The per-row split/concat of the cache (``vrl/models/ar.py:42-110``)
is the identity when all rows advance together and is left out.  The policy stand-in wraps a
real, randomly initialised Hugging Face ``LlamaModel`` like the reference's own stub
(tests/models/test_janus_wrapper.py:30-87).
"""

import types

import pytest
import torch
import torch.nn.functional as F
from torch import nn

from visionrl_amd.ar_decode import StaticARSampler, install_static_ar_sampler

HIDDEN, INTER, HEADS, LAYERS, VOCAB_IMG = 256, 512, 4, 2, 1024


class StubMMGPT(nn.Module):
    def __init__(self, dtype, hidden=HIDDEN, inter=INTER, heads=HEADS, layers=LAYERS, vocab=VOCAB_IMG, kv_heads=None):
        super().__init__()
        from transformers import LlamaConfig, LlamaModel

        cfg = LlamaConfig(hidden_size=hidden, intermediate_size=inter, num_hidden_layers=layers,
                          num_attention_heads=heads, num_key_value_heads=kv_heads or heads, vocab_size=128,
                          max_position_embeddings=1024)
        torch.manual_seed(0)
        self.language_model = types.SimpleNamespace(model=LlamaModel(cfg).to(dtype).eval())
        self.gen_head = nn.Linear(hidden, vocab, bias=False).to(dtype)
        self.gen_embed = nn.Embedding(vocab, hidden).to(dtype)
        with torch.no_grad():   # spread the logits so that draws are not all near-ties
            self.gen_head.weight.mul_(8.0)

    def prepare_gen_img_embeds(self, ids):
        return self.gen_embed(ids)


class StubPolicy:
    def __init__(self, dtype=torch.float32, device="cpu", **shape):
        self.mmgpt = StubMMGPT(dtype, **shape)
        self.mmgpt.language_model.model.to(device)
        self.mmgpt.to(device)
        self.config = types.SimpleNamespace(cfg_weight=5.0, temperature=1.0, image_token_num=12)

    def _base(self):
        return self.mmgpt

    def _lm_trunk(self):
        return self.mmgpt.language_model.model


def make_inputs(B, n_text, dtype, device, seed=3, hidden=HIDDEN, side="left"):
    """Prompt embeddings and masks of a chunk.  ``side="left"``: left padding of different lengths.
    ``side="right"``: what the reference's executor hands over (``_tokenize_prompts`` pads to
    ``max_text_length`` on the right, vrl/models/families/janus_pro/executor.py:439-462, and
    ``align_pair`` right-pads, vrl/engine/ar/executor_base.py:166-195): ones, then zeros, the last
    prompt slot a padding slot, and the unconditional "" prompt of row 0 almost all padding; the image
    tokens' ones follow the zeros, so the mask has a hole in the middle."""
    g = torch.Generator().manual_seed(seed)
    cond = torch.randn(B, n_text, hidden, generator=g).to(dtype).to(device)
    uncond = torch.randn(B, n_text, hidden, generator=g).to(dtype).to(device)
    cmask = torch.ones(B, n_text, dtype=torch.long)
    umask = torch.ones(B, n_text, dtype=torch.long)
    for b in range(B):
        if side == "left":
            cmask[b, :b % 3] = 0
            umask[b, :(b + 2) % 4] = 0
        else:
            cmask[b, n_text - 1 - b % 3:] = 0
            umask[b, (1 if b == 0 else n_text - 1 - (b + 2) % 4):] = 0
    return cond, uncond, cmask.to(device), umask.to(device)


@torch.no_grad()
def reference_loop(policy, cond, uncond, cmask, umask, cfg_weight, temperature, n_img):
    trunk, base = policy._lm_trunk(), policy._base()
    B = cond.shape[0]
    tokens = torch.empty(B, n_img, dtype=torch.long, device=cond.device)
    logprobs = torch.empty(B, n_img, dtype=torch.float32, device=cond.device)
    embeds, attn, past = torch.cat([cond, uncond]), torch.cat([cmask, umask]), None
    for pos in range(n_img):
        out = trunk(inputs_embeds=embeds, attention_mask=attn, use_cache=True, past_key_values=past)
        past = out.past_key_values
        logits = base.gen_head(out.last_hidden_state[:, -1:, :]).squeeze(1)
        c, u = logits.chunk(2, dim=0)
        guided = u + cfg_weight * (c - u)
        probs = F.softmax(guided / temperature, dim=-1)
        sampled = torch.multinomial(probs, num_samples=1).squeeze(-1)
        lp = F.log_softmax(c / temperature, dim=-1).gather(-1, sampled.unsqueeze(-1)).squeeze(-1)
        tokens[:, pos], logprobs[:, pos] = sampled, lp
        embeds = base.prepare_gen_img_embeds(torch.cat([sampled, sampled]).unsqueeze(-1))
        attn = torch.cat([attn, torch.ones(2 * B, 1, dtype=attn.dtype, device=attn.device)], dim=1)
    return tokens, logprobs


# ------------------------------------------------------------------ CPU: the static-cache logic
@pytest.mark.parametrize("side", ["left", "right"])
def test_static_cache_loop_samples_what_the_reference_loop_samples(side):
    policy = StubPolicy()
    cond, uncond, cmask, umask = make_inputs(3, 7, torch.float32, "cpu", side=side)
    assert side == "left" or (int(umask[0].sum()) == 1 and not cmask[:, -1].any())
    torch.manual_seed(11)
    want_t, want_lp = reference_loop(policy, cond, uncond, cmask, umask, 5.0, 1.0, 12)
    sampler = StaticARSampler(policy, graph=False, fused_tail=False)
    torch.manual_seed(11)
    got_t, got_lp = sampler.sample_image_tokens(cond, uncond, cmask, umask)   # defaults from policy.config
    assert got_t.dtype == torch.long and got_lp.dtype == torch.float32 and got_t.shape == (3, 12)
    assert torch.equal(got_t, want_t)
    torch.testing.assert_close(got_lp, want_lp, rtol=1e-5, atol=1e-5)
    assert len(want_t.unique()) > 6   # the draw is not degenerate

    # a second call reuses the buffers (other prompts, other length inside the same bucket, other seed)
    cond2, uncond2, cmask2, umask2 = make_inputs(3, 9, torch.float32, "cpu", seed=4, side=side)
    torch.manual_seed(12)
    want_t2, want_lp2 = reference_loop(policy, cond2, uncond2, cmask2, umask2, 5.0, 1.0, 10)
    torch.manual_seed(12)
    got_t2, got_lp2 = sampler.sample_image_tokens(cond2, uncond2, cmask2, umask2, image_token_num=10)
    assert len(sampler._sessions) == 1
    assert torch.equal(got_t2, want_t2)
    torch.testing.assert_close(got_lp2, want_lp2, rtol=1e-5, atol=1e-5)
    assert torch.equal(got_t, want_t)   # results of the first call are copies, not views of the buffers


def test_guidance_and_temperature_reach_the_draw():
    policy = StubPolicy()
    cond, uncond, cmask, umask = make_inputs(2, 5, torch.float32, "cpu")
    sampler = StaticARSampler(policy, graph=False, fused_tail=False)
    for cfg, temp in ((1.0, 1.0), (7.5, 0.7)):
        torch.manual_seed(5)
        want = reference_loop(policy, cond, uncond, cmask, umask, cfg, temp, 6)
        torch.manual_seed(5)
        got = sampler.sample_image_tokens(cond, uncond, cmask, umask, cfg_weight=cfg, temperature=temp,
                                          image_token_num=6)
        assert torch.equal(got[0], want[0])
        torch.testing.assert_close(got[1], want[1], rtol=1e-5, atol=1e-5)
    assert len(sampler._sessions) == 2   # one per (guidance, temperature): they are baked into a recorded step


def test_contract_violations_raise():
    policy = StubPolicy()
    cond, uncond, cmask, umask = make_inputs(2, 5, torch.float32, "cpu")
    sampler = StaticARSampler(policy, graph=False, fused_tail=False)
    with pytest.raises(ValueError):
        sampler.sample_image_tokens(cond, uncond[:1], cmask, umask)
    with pytest.raises(ValueError):
        sampler.sample_image_tokens(cond, uncond, cmask[:, :4], umask)
    with pytest.raises(ValueError):
        sampler.sample_image_tokens(cond, uncond, cmask, umask, temperature=0.0)
    policy.config = None
    with pytest.raises(ValueError):
        sampler.sample_image_tokens(cond, uncond, cmask, umask)
    with pytest.raises(TypeError):
        StaticARSampler(types.SimpleNamespace(_lm_trunk=policy._lm_trunk, _base=lambda: nn.Identity()))


def test_install_replaces_the_policy_method():
    policy = StubPolicy()
    sampler = install_static_ar_sampler(policy, graph=False, fused_tail=False)
    cond, uncond, cmask, umask = make_inputs(1, 4, torch.float32, "cpu")
    torch.manual_seed(2)
    want = reference_loop(policy, cond, uncond, cmask, umask, 3.0, 1.0, 5)
    torch.manual_seed(2)
    got = policy.sample_image_tokens(cond, uncond, cmask, umask, cfg_weight=3.0, temperature=1.0, image_token_num=5)
    assert torch.equal(got[0], want[0]) and policy._static_ar_sampler is sampler


# ------------------------------------------------------------------ the step API under a token scheduler
class Seq:
    """What ``step_ar`` reads of the scheduler's ``ActiveSequence`` (vrl/engine/ar/sequence.py:21-61)."""

    def __init__(self, row, max_new_tokens):
        self.sample_id, self.metadata, self.position, self.max_new_tokens = f"s{row}", {"row_index": row}, 0, max_new_tokens

    @property
    def finished(self):
        return self.position >= self.max_new_tokens


def scheduled_loop(policy, inputs, n_img, batch_size):
    """The executor's loop (vrl/models/families/janus_pro/executor.py:373-413) with the scheduler's
    grouping (vrl/engine/ar/token_scheduler.py:59-90): first pending position, at most batch_size rows."""
    state = policy.init_ar_state(*inputs, cfg_weight=5.0, temperature=1.0, image_token_num=n_img)
    pending = [Seq(row, n_img) for row in range(inputs[0].shape[0])]
    results = []
    while pending:
        position = pending[0].position
        batch = [seq for seq in pending if seq.position == position][:batch_size]
        results.append(policy.step_ar(state, batch))
        for seq in batch:
            seq.position += 1
        chosen = {id(seq) for seq in batch}
        pending = [seq for seq in pending if id(seq) not in chosen] + [seq for seq in batch if not seq.finished]
    return policy.finalize_ar_state(state), results


def test_step_api_in_lockstep_samples_what_the_reference_loop_samples():
    policy = StubPolicy()
    inputs = make_inputs(3, 6, torch.float32, "cpu", seed=9)
    torch.manual_seed(13)
    want_t, want_lp = reference_loop(policy, *inputs, 5.0, 1.0, 7)
    install_static_ar_sampler(policy, graph=False, fused_tail=False)
    torch.manual_seed(13)
    (got_t, got_lp), results = scheduled_loop(policy, inputs, 7, batch_size=3)
    assert torch.equal(got_t, want_t)
    torch.testing.assert_close(got_lp, want_lp, rtol=1e-5, atol=1e-5)
    assert len(results) == 7
    for p, res in enumerate(results):      # the per-step results carry the same tokens, in row order
        assert res.sequence_ids == ["s0", "s1", "s2"] and res.positions == [p] * 3
        assert torch.equal(res.token, want_t[:, p]) and res.replay_extras == {}
        torch.testing.assert_close(res.log_prob, want_lp[:, p], rtol=1e-5, atol=1e-5)


def test_step_api_contract():
    policy = StubPolicy()
    inputs = make_inputs(3, 6, torch.float32, "cpu", seed=9)
    sampler = install_static_ar_sampler(policy, graph=False, fused_tail=False)
    state = policy.init_ar_state(*inputs, image_token_num=2)
    seqs = [Seq(row, 2) for row in range(3)]
    with pytest.raises(ValueError, match="at least one"):
        policy.step_ar(state, [])
    with pytest.raises(ValueError, match="row indices"):
        policy.step_ar(state, [Seq(7, 2)])
    with pytest.raises(ValueError, match="together"):
        policy.step_ar(state, seqs[:2])                  # this stand-in has no step functions of its own to take over
    seqs[1].position = 1
    with pytest.raises(ValueError, match="positions must match within"):
        policy.step_ar(state, seqs)
    seqs[1].position = 0
    policy.step_ar(state, seqs)
    with pytest.raises(ValueError, match="state's position"):
        policy.step_ar(state, seqs)                      # the sequences were not advanced
    for seq in seqs:
        seq.position = 1
    policy.step_ar(state, seqs)
    for seq in seqs:
        seq.position = 2
    with pytest.raises(ValueError, match="finished"):
        policy.step_ar(state, seqs)
    tokens, logprobs = policy.finalize_ar_state(state)
    assert tokens.shape == (3, 2) and torch.equal(tokens, state.token_ids) and sampler is policy._static_ar_sampler


def test_partial_batches_go_to_the_policys_own_step_functions():
    calls = []

    class WithStepApi(StubPolicy):
        def init_ar_state(self, *args, **kwargs):
            calls.append(("init", kwargs["image_token_num"]))
            return {"steps": 0}

        def step_ar(self, state, sequences, *, generator=None):
            state["steps"] += 1
            calls.append(("step", [seq.metadata["row_index"] for seq in sequences]))
            return "their result"

        def finalize_ar_state(self, state):
            return "their tokens", state["steps"]

    policy = WithStepApi()
    inputs = make_inputs(3, 6, torch.float32, "cpu", seed=9)
    install_static_ar_sampler(policy, graph=False, fused_tail=False)
    final, results = scheduled_loop(policy, inputs, 2, batch_size=2)
    assert final == ("their tokens", 4) and results == ["their result"] * 4
    assert calls == [("init", 2), ("step", [0, 1]), ("step", [2]), ("step", [0, 1]), ("step", [2])]
    # a full batch keeps the static loop, whatever the policy has
    calls.clear()
    torch.manual_seed(1)
    (tokens, _), _ = scheduled_loop(policy, inputs, 2, batch_size=3)
    assert calls == [] and tokens.shape == (3, 2)


# ------------------------------------------------------------------ GPU: int4 modules, fused tail, HIP graph
@pytest.fixture(scope="module")
def int4_policy():
    from visionrl_amd.policy_glue import apply_int4_to_policy

    policy = StubPolicy(torch.bfloat16, "cuda:0")
    summary = apply_int4_to_policy(policy, group_size=128)
    assert summary["prepacked"] > 0 and summary["qkv_groups"] == LAYERS
    return policy


@pytest.mark.gpu
@pytest.mark.parametrize("native", [False, True, "split", "crossing"])
def test_graph_replays_equal_eager_steps(int4_policy, native):
    """Every replayed step against the same step run eagerly: tokens and log-probabilities bit for bit,
    over two calls (the second reuses the recorded graph) with eager work and syncs in between.
    "split": prompts of more than 512 slots, where the attention of few rows divides a pair's slots over several
    workgroups; "crossing": the generation begins below 512 filled slots and ends above, so it is replayed from
    two recordings (one-workgroup launches first, split launches from slot 512 on)."""
    print("ar decode: graph vs eager, native trunk", native, flush=True)
    longer = {"split": 523, "crossing": 492}.get(native, 0)
    form, native = native, bool(native)
    eager = StaticARSampler(int4_policy, graph=False, native=native)
    graphed = StaticARSampler(int4_policy, graph=True, native=native)
    for call, (n_text, n_img, seed) in enumerate(((7 + longer, 24, 21), (11 + longer, 20, 22), (7 + longer, 24, 21))):
        cond, uncond, cmask, umask = make_inputs(3, n_text, torch.bfloat16, "cuda:0", seed=seed)
        torch.manual_seed(seed)
        want_t, want_lp = eager.sample_image_tokens(cond, uncond, cmask, umask, image_token_num=n_img)
        torch.cuda.synchronize()
        torch.manual_seed(seed)
        got_t, got_lp = graphed.sample_image_tokens(cond, uncond, cmask, umask, image_token_num=n_img)
        torch.cuda.synchronize()
        assert torch.equal(got_t, want_t), (call, got_t, want_t)
        assert torch.equal(got_lp, want_lp), call
        assert len(want_t.unique()) > n_img // 2
    (sess,) = graphed._sessions.values()
    assert sess.graph is not None and bool(sess.native) == native
    assert (sess.graph_short is not None) == (form == "crossing")
    if form in ("split", "crossing"):
        assert sess.native.short_form(511) and not sess.native.short_form(512)


@pytest.mark.gpu
def test_short_cache_launch_list_equals_the_default_one(int4_policy, monkeypatch):
    """While no row has 512 filled slots the split launches leave a pair to one workgroup, and the launch list
    with one-workgroup launches in their place does the same arithmetic: same tokens, same log-probabilities
    bit for bit, whichever list the steps run from."""
    print("ar decode: short-cache launch list vs default list", flush=True)
    from visionrl_amd.decode_step import NativeDecodeTrunk
    cond, uncond, cmask, umask = make_inputs(3, 470, torch.bfloat16, "cuda:0", seed=77)
    results = []
    for use_short in (True, False):
        if not use_short:
            monkeypatch.setattr(NativeDecodeTrunk, "short_form", lambda self, cached: False)
        sampler = StaticARSampler(int4_policy, graph=False, native=True)
        torch.manual_seed(5)
        results.append(sampler.sample_image_tokens(cond, uncond, cmask, umask, image_token_num=40))
        torch.cuda.synchronize()
        (sess,) = sampler._sessions.values()
        assert sess.native and sess.native._table_short is not None and sess.max_len == 512
    (t_short, lp_short), (t_long, lp_long) = results
    assert torch.equal(t_short, t_long) and torch.equal(lp_short, lp_long)
    assert len(t_short.unique()) > 20


@pytest.mark.gpu
@pytest.mark.parametrize("side", ["left", "right"])
def test_fused_static_path_samples_what_the_reference_loop_samples(int4_policy, side):
    """Same int4 policy through the reference loop (dynamic cache, torch formulas for the tail):
    same tokens under the same seed; log-probabilities within a bf16 rounding of the log-softmax.
    The trunk stays the module here (``native=False``): the native trunk agrees with it to bf16
    roundings only, which the tests below bound."""
    print("ar decode: static fused vs reference loop", flush=True)
    cond, uncond, cmask, umask = make_inputs(3, 7, torch.bfloat16, "cuda:0", side=side)
    torch.manual_seed(31)
    want_t, want_lp = reference_loop(int4_policy, cond, uncond, cmask, umask, 5.0, 1.0, 16)
    for graph in (False, True):
        torch.manual_seed(31)
        got_t, got_lp = StaticARSampler(int4_policy, graph=graph, native=False).sample_image_tokens(
            cond, uncond, cmask, umask, image_token_num=16)
        torch.cuda.synchronize()
        assert torch.equal(got_t, want_t), (graph, got_t, want_t)
        torch.testing.assert_close(got_lp, want_lp, rtol=2 ** -7, atol=2 ** -7)


@pytest.mark.gpu
@pytest.mark.parametrize("side,split", [("left", False), ("right", False), ("left", True)])
def test_native_trunk_tracks_the_module_trunk(int4_policy, side, split):
    """Teacher-forced: both trunks consume the same inputs step after step, each over its own cache;
    hidden states and appended cache rows stay within bf16 roundings of each other (also with the
    attention in its split form, which long caches of few rows take)."""
    print("ar decode: native trunk vs module trunk", flush=True)
    rows, n_text, steps = 6, 517 if split else 7, 12   # the split form divides a pair from 512 filled slots on
    cond, uncond, cmask, umask = make_inputs(rows // 2, n_text, torch.bfloat16, "cuda:0", seed=41, side=side)
    sessions = []
    for native in (True, False):
        sampler = StaticARSampler(int4_policy, graph=False, native=native)
        torch.manual_seed(41)
        sampler.sample_image_tokens(cond, uncond, cmask, umask, image_token_num=1)   # prompt pass only
        (sess,) = sampler._sessions.values()
        sessions.append((sampler, sess))
    (_, nat), (_, mod) = sessions
    assert nat.native and not mod.native
    assert nat.native.launches == 5 * LAYERS + 1
    trunk = int4_policy._lm_trunk()
    gen = torch.Generator(device="cuda:0").manual_seed(42)
    worst = 0.0
    with torch.no_grad():
        for t in range(steps):
            emb = torch.randn((rows, 1, HIDDEN), generator=gen, device="cuda:0").to(torch.bfloat16)
            nat.cur.copy_(emb)
            got = nat.native.run().float().clone()
            nat.slot.add_(1)
            want = trunk(inputs_embeds=emb, attention_mask=mod.mask, use_cache=True,
                         past_key_values=mod.cache).last_hidden_state[:, -1].float()
            torch.cuda.synchronize()
            err = (got - want).abs()
            worst = max(worst, err.max().item())
            # normalised hidden states are O(1): a few bf16 steps (2^-8 relative) through two layers
            assert err.max().item() <= 0.08 and err.mean().item() <= 0.008, (t, err.max().item(), err.mean().item())
    for layer_n, layer_m in zip(nat.cache.layers, mod.cache.layers):
        for a, b in ((layer_n.keys, layer_m.keys), (layer_n.values, layer_m.values)):
            a, b = a[:, :, :n_text + steps].float(), b[:, :, :n_text + steps].float()
            assert torch.equal(a[:, :, :n_text], b[:, :, :n_text])                 # the prompt pass is shared code
            assert (a - b).abs().max().item() <= 0.05 * b.abs().max().item()
            assert (a[:, :, n_text + steps:] == 0).all()
    print("ar decode: worst hidden-state difference", worst, flush=True)


@pytest.mark.gpu
def test_native_sampling_agrees_with_the_module_path_on_independent_draws(int4_policy):
    """Two image tokens for 16 rows: the first comes from the shared prompt pass (identical), the
    second from one decode step of either trunk under the same noise: draws flip only at near-ties."""
    print("ar decode: native vs module sampling", flush=True)
    cond, uncond, cmask, umask = make_inputs(16, 7, torch.bfloat16, "cuda:0", seed=51)
    out = []
    for native in (True, False):
        torch.manual_seed(52)
        out.append(StaticARSampler(int4_policy, graph=False, native=native).sample_image_tokens(
            cond, uncond, cmask, umask, image_token_num=2))
    torch.cuda.synchronize()
    (t_n, lp_n), (t_m, lp_m) = out
    assert torch.equal(t_n[:, 0], t_m[:, 0]) and torch.equal(lp_n[:, 0], lp_m[:, 0])
    same = t_n[:, 1] == t_m[:, 1]
    assert same.sum().item() >= 14, (t_n[:, 1], t_m[:, 1])
    assert (lp_n[same, 1] - lp_m[same, 1]).abs().max().item() <= 0.25


# ------------------------------------------------------------------ LoRA adapters on the attention projections
class LoraWrapper(nn.Module):
    """The attributes and the forward of peft's ``lora.Linear`` that matter at rollout time
    (``vrl/models/families/janus_pro/policy.py:298-324`` wraps q/k/v/o_proj with it): the frozen
    projection in ``base_layer``, one adapter named "default", the adapter run in its own dtype
    on the upcast input and the sum cast back."""

    def __init__(self, base, r=8, alpha=16, dtype=torch.float32):
        super().__init__()
        self.base_layer = base
        self.lora_A = nn.ModuleDict({"default": nn.Linear(base.in_features, r, bias=False).to(dtype)})
        self.lora_B = nn.ModuleDict({"default": nn.Linear(r, base.out_features, bias=False).to(dtype)})
        self.scaling = {"default": alpha / r}
        self.active_adapters = ["default"]
        self.merged = False
        self.disable_adapters = False
        with torch.no_grad():
            self.lora_B["default"].weight.normal_(0.0, 0.05)   # a trained adapter, not a fresh (zero) one

    def forward(self, x):
        result = self.base_layer(x)
        a, b = self.lora_A["default"], self.lora_B["default"]
        result = result + b(a(x.to(a.weight.dtype))) * self.scaling["default"]
        return result.to(x.dtype)


def lora_policy(dtype):
    from visionrl_amd.policy_glue import apply_int4_to_policy

    policy = StubPolicy(torch.bfloat16, "cuda:0")
    torch.manual_seed(7)
    for layer in policy._lm_trunk().layers:
        for name in ("q_proj", "k_proj", "v_proj", "o_proj"):
            setattr(layer.self_attn, name, LoraWrapper(getattr(layer.self_attn, name), dtype=dtype).to("cuda:0"))
    summary = apply_int4_to_policy(policy, group_size=128)
    assert summary["linears"] == 7 * LAYERS and summary["qkv_groups"] == LAYERS
    return policy


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_native_trunk_with_lora_adapters_tracks_the_module_trunk(dtype):
    """As above with adapters on q/k/v/o: the native layer adds them inside its five launches; a
    weight sync in place (``load_lora_state``) reaches it without rebuilding anything."""
    from visionrl_amd.policy_glue import load_lora_state

    print("ar decode: native trunk with LoRA", dtype, flush=True)
    policy = lora_policy(dtype)
    rows, n_text, steps = 4, 6, 6
    cond, uncond, cmask, umask = make_inputs(rows // 2, n_text, torch.bfloat16, "cuda:0", seed=61)
    sessions = []
    for native in (True, False):
        sampler = StaticARSampler(policy, graph=False, native=native)
        torch.manual_seed(61)
        sampler.sample_image_tokens(cond, uncond, cmask, umask, image_token_num=1)
        (sess,) = sampler._sessions.values()
        sessions.append(sess)
    nat, mod = sessions
    assert nat.native and not mod.native
    assert nat.native.launches == 5 * LAYERS + 1   # the adapters' workgroups of q|k|v normalise their rows themselves
    trunk = policy._lm_trunk()
    gen = torch.Generator(device="cuda:0").manual_seed(62)

    def compare(n):
        with torch.no_grad():
            for t in range(n):
                emb = torch.randn((rows, 1, HIDDEN), generator=gen, device="cuda:0").to(torch.bfloat16)
                nat.cur.copy_(emb)
                got = nat.native.run().float().clone()
                nat.slot.add_(1)
                want = trunk(inputs_embeds=emb, attention_mask=mod.mask, use_cache=True,
                             past_key_values=mod.cache).last_hidden_state[:, -1].float()
                torch.cuda.synchronize()
                err = (got - want).abs()
                assert err.max().item() <= 0.08 and err.mean().item() <= 0.008, (t, err.max().item())
        return got

    before = compare(steps)
    # the adapters matter: without them the hidden states differ by far more than the tolerance
    bare = trunk.layers[0].self_attn.q_proj
    state = {k: torch.randn_like(v) * 0.05 for k, v in trunk.state_dict().items() if "lora_" in k}
    summary = load_lora_state(trunk, state)
    assert summary["loaded"] == 8 * LAYERS
    assert torch.equal(bare.lora_B["default"].weight.data, state["layers.0.self_attn.q_proj.lora_B.default.weight"])
    after = compare(steps)          # same launches, same pointers, new adapter values: still tracks the modules
    assert (after - before).abs().max().item() > 0.1


@pytest.mark.gpu
def test_step_api_with_recorded_steps_equals_sample_image_tokens(int4_policy):
    """The scheduler-driven form over recorded graphs: same tokens as one ``sample_image_tokens`` call,
    twice in a row (the second generation replays from its first decode step on)."""
    print("ar decode: step API over graphs", flush=True)
    inputs = make_inputs(3, 7, torch.bfloat16, "cuda:0", seed=91)
    sampler = StaticARSampler(int4_policy, graph=True)
    holder = types.SimpleNamespace(init_ar_state=sampler.init_ar_state, step_ar=sampler.step_ar,
                                   finalize_ar_state=sampler.finalize_ar_state)
    for seed in (92, 93):
        torch.manual_seed(seed)
        want = StaticARSampler(int4_policy, graph=False).sample_image_tokens(*inputs, image_token_num=9)
        torch.manual_seed(seed)
        got, results = scheduled_loop(holder, inputs, 9, batch_size=3)
        torch.cuda.synchronize()
        assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1])
        assert torch.equal(torch.stack([r.token for r in results], dim=1), want[0])


@pytest.mark.gpu
def test_graph_replays_equal_eager_steps_with_lora():
    print("ar decode: graph vs eager with LoRA", flush=True)
    policy = lora_policy(torch.float32)
    cond, uncond, cmask, umask = make_inputs(2, 7, torch.bfloat16, "cuda:0", seed=71)
    out = []
    for graph in (False, True):
        torch.manual_seed(71)
        out.append(StaticARSampler(policy, graph=graph).sample_image_tokens(cond, uncond, cmask, umask,
                                                                             image_token_num=16))
    torch.cuda.synchronize()
    assert torch.equal(out[0][0], out[1][0]) and torch.equal(out[0][1], out[1][1])


# ------------------------------------------------------------------ the real layer shapes
@pytest.mark.gpu
@pytest.mark.parametrize("B,kv_heads,lora,hidden,inter,heads", [
    (1, 16, False, 2048, 5632, 16), (16, 16, False, 2048, 5632, 16), (16, 4, True, 2048, 5632, 16),
    (1, 32, False, 4096, 11008, 32), (16, 32, True, 4096, 11008, 32),      # the 7B-class layer
    (24, 16, False, 2048, 5632, 16), (32, 4, False, 2048, 5632, 16),       # 48 and 64 rows: two launches per linear
])
def test_native_trunk_at_janus_layer_shapes(B, kv_heads, lora, hidden, inter, heads):
    """Two decoder layers of the Janus-Pro-1B geometry (2048 hidden, 16 heads of 128, 5632 intermediate,
    16384 image tokens) and of the 7B-class one (4096, 32 heads, 11008): the 128-wide heads, the row
    slabs of down_proj, the 32-row launches and the 4096-wide normalising launches are on the path here.  Native trunk against module trunk (teacher-forced), recorded graph against eager
    steps, and the same seed sampling the same tokens twice (what the reference's own determinism test
    asks of the loop, tests/engine/generation/test_pipeline_janus_pro.py:337-400)."""
    from visionrl_amd.policy_glue import apply_int4_to_policy

    print("ar decode: Janus layer shapes", B, kv_heads, lora, hidden, inter, heads, flush=True)
    policy = StubPolicy(torch.bfloat16, "cuda:0", hidden=hidden, inter=inter, heads=heads, layers=2, vocab=16384,
                        kv_heads=kv_heads)
    if lora:
        torch.manual_seed(5)
        for layer in policy._lm_trunk().layers:
            for name in ("q_proj", "k_proj", "v_proj", "o_proj"):
                setattr(layer.self_attn, name,
                        LoraWrapper(getattr(layer.self_attn, name), r=32, alpha=64).to("cuda:0"))
    apply_int4_to_policy(policy, group_size=128)
    rows, n_text, steps = 2 * B, 40, 5
    cond, uncond, cmask, umask = make_inputs(B, n_text, torch.bfloat16, "cuda:0", seed=81, hidden=hidden)
    sessions = []
    for native in (True, False):
        sampler = StaticARSampler(policy, graph=False, native=native)
        torch.manual_seed(81)
        sampler.sample_image_tokens(cond, uncond, cmask, umask, image_token_num=1)
        (sess,) = sampler._sessions.values()
        sessions.append(sess)
    nat, mod = sessions
    assert nat.native and not mod.native
    trunk = policy._lm_trunk()
    gen = torch.Generator(device="cuda:0").manual_seed(82)
    with torch.no_grad():
        for t in range(steps):
            emb = torch.randn((rows, 1, hidden), generator=gen, device="cuda:0").to(torch.bfloat16)
            nat.cur.copy_(emb)
            got = nat.native.run().float().clone()
            nat.slot.add_(1)
            want = trunk(inputs_embeds=emb, attention_mask=mod.mask, use_cache=True,
                         past_key_values=mod.cache).last_hidden_state[:, -1].float()
            torch.cuda.synchronize()
            err = (got - want).abs()
            assert err.max().item() <= 0.1 and err.mean().item() <= 0.008, (t, err.max().item(), err.mean().item())
    del sessions, nat, mod
    out = []
    for graph in (False, True, True):
        torch.manual_seed(83)
        out.append(StaticARSampler(policy, graph=graph).sample_image_tokens(cond, uncond, cmask, umask,
                                                                             image_token_num=10))
    torch.cuda.synchronize()
    for tokens, logprobs in out[1:]:
        assert torch.equal(tokens, out[0][0]) and torch.equal(logprobs, out[0][1])
    assert out[0][0].shape == (B, 10) and (out[0][0] >= 0).all() and (out[0][0] < 16384).all()
    assert (out[0][1] <= 0).all() and torch.isfinite(out[0][1]).all()


@pytest.mark.gpu
def test_adapter_state_changes_invalidate_the_recorded_step():
    """Disabling the adapters (what the policy's reference-policy context does, policy.py:21) between two
    generations: the second one must not replay a step recorded with them."""
    print("ar decode: adapter state change", flush=True)
    policy = lora_policy(torch.float32)
    inputs = make_inputs(2, 7, torch.bfloat16, "cuda:0", seed=95)
    sampler = StaticARSampler(policy, graph=True)
    torch.manual_seed(96)
    with_adapters = sampler.sample_image_tokens(*inputs, image_token_num=8)
    (sess,) = sampler._sessions.values()
    first_graph = sess.graph
    assert sess.native and first_graph is not None
    wrappers = [getattr(layer.self_attn, n) for layer in policy._lm_trunk().layers
                for n in ("q_proj", "k_proj", "v_proj", "o_proj")]

    for w in wrappers:
        w.disable_adapters = True
        w.forward = types.MethodType(lambda self, x: self.base_layer(x), w)
    torch.manual_seed(96)
    without = sampler.sample_image_tokens(*inputs, image_token_num=8)
    torch.cuda.synchronize()
    assert sess.graph is not first_graph and not sess.native   # disabled adapters: this stand-in keeps the module path
    torch.manual_seed(96)
    want = StaticARSampler(policy, graph=False, native=False).sample_image_tokens(*inputs, image_token_num=8)
    assert torch.equal(without[0], want[0]) and torch.equal(without[1], want[1])
    assert not torch.equal(without[1], with_adapters[1])


# ------------------------------------------------------------------ the checkpoints' two-layer head and aligner
class VisionHead(nn.Module):
    """``gen_head`` as the Janus-Pro checkpoints hold it (the ``vision_head`` class of the upstream package, which
    ``vrl/models/families/janus_pro/policy.py:803-842`` loads and ``policy.py:138-160`` calls): Linear, GELU,
    Linear, both linears with a bias."""

    def __init__(self, hidden, vocab):
        super().__init__()
        self.output_mlp_projector = nn.Linear(hidden, hidden)
        self.vision_activation = nn.GELU()
        self.vision_head = nn.Linear(hidden, vocab)

    def forward(self, x):
        return self.vision_head(self.vision_activation(self.output_mlp_projector(x)))


class JanusShapedMMGPT(StubMMGPT):
    """The stub with the checkpoints' head and input path of image tokens: ``gen_embed`` (8 values per token)
    and the two-layer ``gen_aligner`` behind ``prepare_gen_img_embeds``."""

    def __init__(self, dtype, aligner=True, **shape):
        super().__init__(dtype, **shape)
        hidden, vocab = shape.get("hidden", HIDDEN), shape.get("vocab", VOCAB_IMG)
        torch.manual_seed(5)
        self.gen_head = VisionHead(hidden, vocab).to(dtype)
        with torch.no_grad():
            self.gen_head.vision_head.weight.mul_(24.0)
            self.gen_head.vision_head.bias.normal_(0.0, 1.0)
            self.gen_head.output_mlp_projector.bias.normal_(0.0, 0.5)
        if aligner:
            self.gen_embed = nn.Embedding(vocab, 8).to(dtype)
            self.gen_aligner = nn.Sequential(nn.Linear(8, hidden), nn.GELU(), nn.Linear(hidden, hidden)).to(dtype)

    def prepare_gen_img_embeds(self, ids):
        embeds = self.gen_embed(ids)
        return self.gen_aligner(embeds) if hasattr(self, "gen_aligner") else embeds


def janus_shaped_policy(aligner=True):
    from visionrl_amd.policy_glue import apply_int4_to_policy

    policy = StubPolicy(torch.bfloat16, "cuda:0")
    policy.mmgpt = JanusShapedMMGPT(torch.bfloat16, aligner=aligner)
    policy.mmgpt.language_model.model.to("cuda:0")
    policy.mmgpt.to("cuda:0")
    summary = apply_int4_to_policy(policy, group_size=128)
    assert summary["head_linears"] == 2          # both linears of the head, found below its attributes
    head = policy.mmgpt.gen_head
    assert head.vision_head._packed is not None and head.output_mlp_projector._packed is not None
    assert head.vision_head.bias is not None and head.output_mlp_projector.bias is not None
    return policy


@pytest.mark.gpu
@pytest.mark.parametrize("aligner", [False, True])
def test_two_layer_head_runs_as_two_launches_and_samples_what_the_module_head_samples(aligner):
    """The checkpoints' head through ``apply_int4_to_policy`` and the static sampler: its front is one launch
    (final norm while staging, bias, GELU), its last linear and the tail one call; tokens under one seed equal
    those of the same sampler with the head as modules followed by ``cfg_sample`` (and of eager steps), the
    log-probabilities agree to a bf16 step."""
    print("ar decode: two-layer head, aligner", aligner, flush=True)
    policy = janus_shaped_policy(aligner)
    cond, uncond, cmask, umask = make_inputs(3, 7, torch.bfloat16, "cuda:0", seed=61)
    runs = {}
    for name, opts in (("fused", {}), ("fused_eager", {"graph": False}), ("modules", {"fused_head": False}),
                       ("no_table", {"embed_table": False})):
        sampler = StaticARSampler(policy, **opts)
        torch.manual_seed(62)
        runs[name] = sampler.sample_image_tokens(cond, uncond, cmask, umask, image_token_num=24)
        torch.cuda.synchronize()
        (sess,) = sampler._sessions.values()
        assert sess.native, name
        if name == "fused":
            assert sess.front_call is not None and sess.native.final is not None and sess.graph is not None
            assert sess.native.launches == 5 * LAYERS        # the last norm went into the head's front launch
            if not aligner:
                assert sampler._table is not None            # a plain embedding tabulates exactly
        if name == "modules":
            assert sess.front_call is None and sess.native.launches == 5 * LAYERS + 1
        if name == "no_table":
            assert sampler._table is None
    want_t, want_lp = runs["modules"]
    assert len(want_t.unique()) > 12
    for name in ("fused", "fused_eager", "no_table"):
        got_t, got_lp = runs[name]
        assert torch.equal(got_t, want_t), (name, got_t, want_t)
        torch.testing.assert_close(got_lp, want_lp, rtol=2 ** -7, atol=2 ** -7)
    assert torch.equal(runs["fused"][1], runs["fused_eager"][1])


@pytest.mark.gpu
def test_two_layer_head_logits_against_the_oracle():
    """The head's two launches against the oracle's arithmetic on the same operands: front = GELU(bf16(x . W1^T)
    + b1) with the stated roundings, logits = bf16(front . W2^T) + b2."""
    import numpy as np

    from oracle import int4_oracle as o
    from tests._util import bf16_to_bits

    print("ar decode: two-layer head against the oracle", flush=True)
    policy = janus_shaped_policy(False)
    head = policy.mmgpt.gen_head
    from visionrl_amd import ops

    x = torch.randn((6, HIDDEN), device="cuda:0").to(torch.bfloat16)
    front = ops.EpilogueGemv(x, head.output_mlp_projector._packed, head.output_mlp_projector.bias, gelu=True).launch()
    logits = torch.empty((6, VOCAB_IMG), dtype=torch.bfloat16, device="cuda:0")
    ops.head_sample(front, head.vision_head._packed, 5.0, 1.0, logits_out=logits, bias=head.vision_head.bias)
    torch.cuda.synchronize()
    assert torch.equal(logits.view(6, 1, -1), head(x.view(6, 1, -1)))          # the module path, bit for bit

    def lin(mod, xin_bits):
        args = (xin_bits, mod.qweight.cpu().numpy(), bf16_to_bits(mod.scales), mod.qzeros.cpu().numpy(), 128)
        y_ref, a_ref = o.gemv_and_abs_f64(*args)
        return y_ref, a_ref, o.bf16_bits_to_f32(bf16_to_bits(mod.bias)).astype(np.float64)

    y1, a1, b1 = lin(head.output_mlp_projector, bf16_to_bits(x))
    pre = o.bf16_bits_to_f32(o.f32_to_bf16_bits((o.bf16_bits_to_f32(o.f32_to_bf16_bits(y1.astype(np.float32))) + b1).astype(np.float32)))
    from math import erf
    gelu = np.vectorize(lambda v: 0.5 * v * (1.0 + erf(v / np.sqrt(2.0))))
    # the front launch within the linear's tolerance carried through bias and GELU (slope at most 1.13)
    got_front = o.bf16_bits_to_f32(bf16_to_bits(front)).astype(np.float64)
    tol = 1.13 * o.gemv_tolerance(y1, a1) + 2.0 ** -7 * np.abs(gelu(y1 + b1)) + 2.0 ** -8 * np.abs(y1 + b1) + 1e-30
    assert (np.abs(got_front - gelu(y1 + b1)) <= tol).all()
    # the last linear over the launch's own front output
    y2, a2, b2 = lin(head.vision_head, bf16_to_bits(front))
    got = o.bf16_bits_to_f32(bf16_to_bits(logits)).astype(np.float64)
    # the linear's tolerance, and one more bf16 rounding for the sum with the bias
    assert (np.abs(got - (y2 + b2)) <= o.gemv_tolerance(y2, a2) + o.bf16_ulp(y2 + b2)).all()


# ------------------------------------------------------------------ partial scheduler batches over the static cache
@pytest.mark.gpu
@pytest.mark.parametrize("head,batch_size", [("linear", 2), ("two_layer", 2), ("linear", 4)])
def test_partial_batches_run_over_the_static_cache(int4_policy, head, batch_size, monkeypatch):
    """A token scheduler that steps fewer rows than the chunk holds (``policy.py:631-645`` with ``row_indices``;
    the reference cuts those rows out of its per-row caches, ``vrl/models/ar.py:42-110``): on the native path the
    rows keep one static cache and a slot counter each.  Rows are independent given their draws, so the result
    must be, bit for bit, what the same sampler gives when it steps every row together with the very draws the
    partial batches used (recorded in the first run, injected in the second), and the draws are made per batch,
    in the order of its rows, as ``torch.multinomial`` would make them for those rows alone."""
    from visionrl_amd import ops

    print("ar decode: partial scheduler batches,", head, batch_size, flush=True)
    policy = int4_policy if head == "linear" else janus_shaped_policy(False)
    B, n_img = 5, 9
    inputs = make_inputs(B, 7, torch.bfloat16, "cuda:0", seed=71)
    vocab = VOCAB_IMG
    original = ops.head_sample
    calls = []

    def recording(x, packed, w, t, **kw):
        calls.append((kw["active"].clone(), kw["noise"].clone()))
        return original(x, packed, w, t, **kw)

    monkeypatch.setattr(ops, "head_sample", recording)
    sampler = install_static_ar_sampler(policy, graph=False)
    torch.manual_seed(72)
    (got_t, got_lp), results = scheduled_loop(policy, inputs, n_img, batch_size=batch_size)
    torch.cuda.synchronize()
    groups = [list(range(g, min(B, g + batch_size))) for g in range(0, B, batch_size)]
    assert len(results) == n_img * len(groups) and len(calls) == len(results)
    (sess,) = sampler._sessions.values()
    assert sess.native_rows is not None and sess.native_rows.launches == 5 * LAYERS + 1
    assert got_t.shape == (B, n_img) and int(sess.pos_rows.min()) == n_img and int(sess.pos_rows.max()) == n_img
    assert sess.slot_rows.tolist() == [7 + n_img - 1] * (2 * B)
    # the draws were made batch by batch, for the rows of the batch only, continuing one random stream
    torch.manual_seed(72)
    step = 0
    assembled = torch.ones((n_img, B, vocab), dtype=torch.bfloat16, device="cuda:0")
    for p in range(n_img):
        for rows in groups:
            active, noise = calls[step]
            assert active.tolist() == [1 if r in rows else 0 for r in range(B)]
            want = torch.empty((len(rows), vocab), dtype=torch.bfloat16, device="cuda:0").exponential_(1.0)
            assert torch.equal(noise[rows], want)
            assembled[p, rows] = want
            res = results[step]
            assert res.positions == [p] * len(rows) and res.sequence_ids == [f"s{r}" for r in rows]
            assert torch.equal(res.token, got_t[rows, p]) and torch.equal(res.log_prob, got_lp[rows, p])
            step += 1
    # the same draws, every row stepped together
    k = [0]

    def injecting(x, packed, w, t, **kw):
        kw["noise"] = assembled[k[0]].contiguous()
        k[0] += 1
        return original(x, packed, w, t, **kw)

    monkeypatch.setattr(ops, "head_sample", injecting)
    together = StaticARSampler(policy, graph=False)
    want_t, want_lp = together.sample_image_tokens(*inputs, cfg_weight=5.0, temperature=1.0, image_token_num=n_img)
    torch.cuda.synchronize()
    assert k[0] == n_img and len(want_t.unique()) > n_img
    assert torch.equal(got_t, want_t)
    if head == "linear":
        assert torch.equal(got_lp, want_lp)
    else:   # stepping all rows together, the head's front is one launch with the last norm folded in
        torch.testing.assert_close(got_lp, want_lp, rtol=2 ** -7, atol=2 ** -7)


@pytest.mark.gpu
def test_a_partial_batch_after_steps_of_the_whole_chunk(int4_policy):
    """The scheduler may narrow its batch in the middle of a generation: the shared counters become one per row
    where they stand, and the rows go on from there; repeated finalize calls return the same tokens."""
    print("ar decode: whole-chunk steps, then partial batches", flush=True)
    B, n_img = 4, 6
    inputs = make_inputs(B, 7, torch.bfloat16, "cuda:0", seed=81)
    install_static_ar_sampler(int4_policy, graph=True)
    state = int4_policy.init_ar_state(*inputs, cfg_weight=5.0, temperature=1.0, image_token_num=n_img)
    seqs = [Seq(r, n_img) for r in range(B)]
    torch.manual_seed(82)
    for _ in range(3):
        int4_policy.step_ar(state, seqs)
        for seq in seqs:
            seq.position += 1
    head_tokens = state.token_ids[:, :3].clone()
    for p in range(3, n_img):
        for rows in ([0, 1, 2], [3]):
            batch = [seqs[r] for r in rows]
            res = int4_policy.step_ar(state, batch)
            assert res.positions == [p] * len(rows)
            for seq in batch:
                seq.position += 1
    with pytest.raises(ValueError, match="finished"):
        int4_policy.step_ar(state, [seqs[0]])
    seqs[1].position = 2
    with pytest.raises(ValueError, match="does not match"):
        int4_policy.step_ar(state, [seqs[1]])                 # the sequence lags behind its row
    tokens, logprobs = int4_policy.finalize_ar_state(state)
    torch.cuda.synchronize()
    assert state.finished and tokens.shape == (B, n_img) and torch.equal(tokens[:, :3], head_tokens)
    assert bool((tokens >= 0).all()) and bool((tokens < VOCAB_IMG).all()) and bool((logprobs <= 0).all())
    again = int4_policy.finalize_ar_state(state)
    assert torch.equal(again[0], tokens) and torch.equal(again[1], logprobs)


@pytest.mark.gpu
def test_recording_keeps_the_garbage_collector_out_and_sessions_die_with_their_sampler(int4_policy, monkeypatch):
    """A finalizer that frees device resources in the middle of a stream capture ends the process: the cyclic
    collector is off while a step is recorded (and back on afterwards), and a sampler holds its sessions without a
    reference cycle, so dropping it frees them (their recorded graphs included) at once."""
    import gc
    import weakref

    from visionrl_amd import ar_decode

    print("ar decode: no garbage collection inside a recording", flush=True)
    seen = []
    step = ar_decode._Session.step

    def watched(self, *args):
        if torch.cuda.is_current_stream_capturing():
            seen.append(gc.isenabled())
        return step(self, *args)

    monkeypatch.setattr(ar_decode._Session, "step", watched)
    cond, uncond, cmask, umask = make_inputs(2, 6, torch.bfloat16, "cuda:0", seed=81)
    sampler = StaticARSampler(int4_policy)
    assert gc.isenabled()
    sampler.sample_image_tokens(cond, uncond, cmask, umask, image_token_num=6)
    torch.cuda.synchronize()
    assert seen == [False] and gc.isenabled()
    (sess,) = sampler._sessions.values()
    assert sess.graph is not None
    gone = weakref.ref(sess)
    del sess
    gc.disable()
    try:
        del sampler
        assert gone() is None        # freed by reference counting alone
    finally:
        gc.enable()
