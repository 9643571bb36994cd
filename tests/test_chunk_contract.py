"""The chunk-level caller of the sampling path, driven through the installed static sampler.

``ChunkDriver`` restates what ``JanusProPipelineExecutor.forward_chunk`` and ``forward`` do around the
sampling call (vrl/models/families/janus_pro/executor.py:254-328, :135-252, scheduler path :340-413):
seed the global generator (``seed + chunk offset``), tokenise the prompt ``sample_count`` times and as
many empty unconditional prompts to ``[B, max_text_length]`` ids and masks, embed both halves, sample
``image_token_num`` tokens either through ``policy.sample_image_tokens`` or through the step API under
the token scheduler's grouping (vrl/engine/ar/token_scheduler.py:59-90), and hand back ids,
log-probabilities and a mask of ones.  The reference itself is not imported; the facts asserted are the
ones its own tests pin at this level: shapes and dtypes, ``lp <= 0``, ids inside the image vocabulary
(tests/models/test_janus_wrapper.py:142-175), bitwise repeatability under a seed with the scheduler
off, on, and on with partial batches (tests/engine/generation/test_pipeline_janus_pro.py:337-400).
"""

import types

import pytest
import torch
from torch import nn

from tests.test_ar_decode import HIDDEN, VOCAB_IMG, Seq, StubPolicy, reference_loop
from visionrl_amd.ar_decode import install_static_ar_sampler

TEXT_VOCAB, PAD_ID, MAX_TEXT = 96, 0, 256
IMAGE_TOKENS = 576


class ChunkDriver:
    """The executor's side of one chunk.  ``padding`` is the tokenizer's padding side."""

    def __init__(self, policy, device="cpu", dtype=torch.float32, padding="left"):
        self.policy, self.device, self.padding = policy, device, padding
        torch.manual_seed(5)
        self.embed = nn.Embedding(TEXT_VOCAB, HIDDEN).to(dtype).to(device)   # language_model.get_input_embeddings()

    def tokenize(self, prompts):
        ids = torch.full((len(prompts), MAX_TEXT), PAD_ID, dtype=torch.long)
        mask = torch.zeros((len(prompts), MAX_TEXT), dtype=torch.long)
        for b, prompt in enumerate(prompts):
            toks = [1] + [2 + (ord(ch) * 7 + i) % (TEXT_VOCAB - 2) for i, ch in enumerate(prompt)][:MAX_TEXT - 2] + [1]
            if self.padding == "left":
                ids[b, MAX_TEXT - len(toks):] = torch.tensor(toks)
                mask[b, MAX_TEXT - len(toks):] = 1
            else:
                ids[b, :len(toks)] = torch.tensor(toks)
                mask[b, :len(toks)] = 1
        return ids.to(self.device), mask.to(self.device)

    @torch.no_grad()
    def forward_chunk(self, prompt, sample_count, *, seed, chunk_offset=0, image_token_num=IMAGE_TOKENS,
                      cfg_weight=5.0, temperature=1.0, use_ar_scheduler=False, ar_scheduler_batch_size=None):
        torch.manual_seed(seed + chunk_offset)
        prompt_ids, prompt_mask = self.tokenize([prompt] * sample_count)
        uncond_ids, uncond_mask = self.tokenize([""] * sample_count)
        cond, uncond = self.embed(prompt_ids), self.embed(uncond_ids)
        kwargs = dict(cfg_weight=cfg_weight, temperature=temperature, image_token_num=image_token_num)
        if use_ar_scheduler:
            state = self.policy.init_ar_state(cond, uncond, prompt_mask, uncond_mask, **kwargs)
            pending = [Seq(row, image_token_num) for row in range(sample_count)]
            batch_size = ar_scheduler_batch_size or sample_count
            while pending:
                position = pending[0].position
                batch = [seq for seq in pending if seq.position == position][:batch_size]
                self.policy.step_ar(state, batch)
                for seq in batch:
                    seq.position += 1
                chosen = {id(seq) for seq in batch}
                pending = [s for s in pending if id(s) not in chosen] + [s for s in batch if not s.finished]
            token_ids, log_probs = self.policy.finalize_ar_state(state)
        else:
            token_ids, log_probs = self.policy.sample_image_tokens(cond, uncond, prompt_mask, uncond_mask, **kwargs)
        return types.SimpleNamespace(token_ids=token_ids, token_log_probs=log_probs,
                                     token_mask=torch.ones_like(log_probs), prompt_attention_mask=prompt_mask,
                                     uncond_attention_mask=uncond_mask, cond=cond, uncond=uncond)


def assert_chunk_facts(out, B, n_img, device):
    assert out.token_ids.shape == (B, n_img) and out.token_log_probs.shape == (B, n_img)
    assert out.token_ids.dtype == torch.long and out.token_log_probs.dtype == torch.float32
    assert out.token_mask.shape == (B, n_img) and out.token_mask.dtype == torch.float32 and bool((out.token_mask == 1).all())
    assert out.token_ids.device.type == torch.device(device).type
    assert bool((out.token_log_probs <= 0).all()) and bool(torch.isfinite(out.token_log_probs).all())
    assert bool((out.token_ids >= 0).all()) and bool((out.token_ids < VOCAB_IMG).all())
    assert out.prompt_attention_mask.shape == (B, MAX_TEXT) and out.uncond_attention_mask.shape == (B, MAX_TEXT)


@pytest.mark.parametrize("padding", ["left", "right"])
def test_forward_chunk_through_the_installed_sampler(padding):
    """A 576-token image for a 3-sample chunk over [3, 256] prompts, on the CPU: the facts the
    reference's tests pin, the reference loop's tokens under the same seed, and repeatability with a
    second, identically built policy, with the scheduler off and on."""
    n_img = IMAGE_TOKENS
    policy = StubPolicy()
    install_static_ar_sampler(policy, graph=False, fused_tail=False)
    driver = ChunkDriver(policy, padding=padding)
    out = driver.forward_chunk("a red cube on a blue sphere", 3, seed=1234, chunk_offset=2)
    assert_chunk_facts(out, 3, n_img, "cpu")
    # the unconditional "" prompt is two tokens: its rows are almost all padding
    assert int(out.uncond_attention_mask[0].sum()) == 2
    assert bool(out.prompt_attention_mask[0, -1 if padding == "left" else 0])
    assert len(out.token_ids.unique()) > 100

    # what the reference's loop samples for this chunk (same seed, dynamic cache, torch formulas)
    plain = StubPolicy()
    torch.manual_seed(1234 + 2)
    want_t, want_lp = reference_loop(plain, out.cond, out.uncond, out.prompt_attention_mask,
                                     out.uncond_attention_mask, 5.0, 1.0, n_img)
    assert torch.equal(out.token_ids, want_t)
    torch.testing.assert_close(out.token_log_probs, want_lp, rtol=1e-5, atol=2e-5)

    # bitwise repeatability: another policy built alike, scheduler on (all rows per step)
    policy_b = StubPolicy()
    install_static_ar_sampler(policy_b, graph=False, fused_tail=False)
    out_b = ChunkDriver(policy_b, padding=padding).forward_chunk("a red cube on a blue sphere", 3, seed=1234,
                                                                 chunk_offset=2, use_ar_scheduler=True)
    assert_chunk_facts(out_b, 3, n_img, "cpu")
    assert torch.equal(out.token_ids, out_b.token_ids) and torch.equal(out.token_log_probs, out_b.token_log_probs)
    # another chunk offset is another stream
    out_c = driver.forward_chunk("a red cube on a blue sphere", 3, seed=1234, chunk_offset=3, image_token_num=8)
    assert not torch.equal(out_c.token_ids, out.token_ids[:, :8])


def test_partial_scheduler_batches_are_repeatable_and_complete():
    """``ar_scheduler_batch_size`` below the chunk size: the generation goes to the policy's own step
    functions (rows at different positions need per-row caches); every row still gets all its tokens
    and two runs under one seed agree bit for bit."""

    class WithStepApi(StubPolicy):
        """Step functions in the reference's shape over its black-box loop: one row at a time."""

        def init_ar_state(self, cond, uncond, cmask, umask, *, cfg_weight, temperature, image_token_num):
            torch_state = torch.random.get_rng_state()
            rows = []
            for b in range(cond.shape[0]):
                torch.random.set_rng_state(torch_state)
                torch.manual_seed(int(torch.initial_seed()) + b)
                rows.append(reference_loop(self, cond[b:b + 1], uncond[b:b + 1], cmask[b:b + 1], umask[b:b + 1],
                                           cfg_weight, temperature, image_token_num))
            return {"tokens": torch.cat([t for t, _ in rows]), "lps": torch.cat([lp for _, lp in rows]), "steps": 0}

        def step_ar(self, state, sequences, *, generator=None):
            state["steps"] += 1
            return None

        def finalize_ar_state(self, state):
            return state["tokens"], state["lps"]

    outs = []
    for _ in range(2):
        policy = WithStepApi()
        install_static_ar_sampler(policy, graph=False, fused_tail=False)
        driver = ChunkDriver(policy)
        outs.append(driver.forward_chunk("two cats", 5, seed=77, image_token_num=6, use_ar_scheduler=True,
                                         ar_scheduler_batch_size=2))
        assert_chunk_facts(outs[-1], 5, 6, "cpu")
    assert torch.equal(outs[0].token_ids, outs[1].token_ids)
    assert torch.equal(outs[0].token_log_probs, outs[1].token_log_probs)


def test_two_live_generations_of_one_shape_do_not_share_buffers():
    """The reference's states are independent objects (policy.py:114-130): a second ``init_ar_state``
    before the first generation is finalized must not hand out the same cache and token buffers."""
    policy = StubPolicy()
    sampler = install_static_ar_sampler(policy, graph=False, fused_tail=False)
    driver = ChunkDriver(policy)
    ids, mask = driver.tokenize(["left", "right"])
    uids, umask = driver.tokenize(["", ""])
    with torch.no_grad():
        cond, uncond = driver.embed(ids), driver.embed(uids)
    plain = StubPolicy()
    wants = []
    for seed in (3, 4):
        torch.manual_seed(seed)
        wants.append(reference_loop(plain, cond, uncond, mask, umask, 5.0, 1.0, 4))
    a = policy.init_ar_state(cond, uncond, mask, umask, image_token_num=4)
    b = policy.init_ar_state(cond, uncond, mask, umask, image_token_num=4)
    assert a.session is not b.session
    seqs_a, seqs_b = [Seq(r, 4) for r in range(2)], [Seq(r, 4) for r in range(2)]
    rng = {}
    for name, seed in (("a", 3), ("b", 4)):
        torch.manual_seed(seed)
        rng[name] = torch.random.get_rng_state()
    for _ in range(4):      # the two generations interleaved, each on its own random stream
        for name, state, seqs in (("a", a, seqs_a), ("b", b, seqs_b)):
            torch.random.set_rng_state(rng[name])
            policy.step_ar(state, seqs)
            rng[name] = torch.random.get_rng_state()
            for seq in seqs:
                seq.position += 1
    tok_a = a.token_ids
    got_a, got_b = policy.finalize_ar_state(a), policy.finalize_ar_state(b)
    assert torch.equal(got_a[0], wants[0][0]) and torch.equal(got_b[0], wants[1][0])
    # finished states hand out copies, and a finalized session serves the next generation of the shape
    c = policy.init_ar_state(cond, uncond, mask, umask, image_token_num=4)
    assert c.session in (a.session, b.session) and len(sampler._sessions) == 1
    torch.manual_seed(9)
    policy.step_ar(c, [Seq(r, 4) for r in range(2)])
    assert torch.equal(tok_a, wants[0][0]) and torch.equal(a.token_ids, wants[0][0])
    # like the reference's (policy.py:616-622), a second finalize returns the same results
    again = policy.finalize_ar_state(a)
    assert torch.equal(again[0], wants[0][0]) and torch.equal(again[1], got_a[1])


@pytest.mark.gpu
@pytest.mark.parametrize("padding", ["left", "right"])
def test_forward_chunk_on_the_int4_policy(padding):
    """The same chunk on the device over the int4 policy, native trunk, fused tail, recorded steps:
    a 576-token image for 3 samples; repeatable bit for bit, scheduler on or off, and equal to the
    same sampler stepping eagerly."""
    from visionrl_amd.policy_glue import apply_int4_to_policy

    dev = "cuda:0"
    print("chunk contract on the int4 policy,", padding, "padding", flush=True)
    policy = StubPolicy(torch.bfloat16, dev)
    apply_int4_to_policy(policy, group_size=128)
    sampler = install_static_ar_sampler(policy)
    driver = ChunkDriver(policy, dev, torch.bfloat16, padding)
    out = driver.forward_chunk("a red cube on a blue sphere", 3, seed=1234, chunk_offset=1)
    torch.cuda.synchronize()
    assert_chunk_facts(out, 3, IMAGE_TOKENS, dev)
    (sess,) = sampler._sessions.values()
    assert sess.native and sess.graph is not None
    again = driver.forward_chunk("a red cube on a blue sphere", 3, seed=1234, chunk_offset=1, use_ar_scheduler=True)
    torch.cuda.synchronize()
    assert torch.equal(out.token_ids, again.token_ids) and torch.equal(out.token_log_probs, again.token_log_probs)
    eager_policy = StubPolicy(torch.bfloat16, dev)
    apply_int4_to_policy(eager_policy, group_size=128)
    install_static_ar_sampler(eager_policy, graph=False)
    eager = ChunkDriver(eager_policy, dev, torch.bfloat16, padding).forward_chunk(
        "a red cube on a blue sphere", 3, seed=1234, chunk_offset=1)
    torch.cuda.synchronize()
    assert torch.equal(out.token_ids, eager.token_ids) and torch.equal(out.token_log_probs, eager.token_log_probs)
    assert len(out.token_ids.unique()) > 100
