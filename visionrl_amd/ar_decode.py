"""Image-token sampling over a static KV cache, one HIP graph replay per decode step.

Stands for ``JanusProPolicy.sample_image_tokens`` (``vrl/models/families/janus_pro/policy.py:476-525``)
and the step it loops over (``_sample_ar_step``, ``policy.py:624-731``), with the same
arguments, the same results and the same use of the random stream:

* The reference keeps one KV cache per row, concatenates the rows before every trunk call and
  splits them afterwards (``policy.py:664-682``, ``vrl/models/ar.py:42-110``: a copy of the whole
  cache per token), rebuilds the attention masks with ``torch.cat`` (``policy.py:701-720``) and
  reads row positions back to the host twice per token (``policy.py:638``, ``:730``).  When all
  rows advance together, as they do in ``sample_image_tokens``, split-then-concat is the identity
  and the positions are known on the host, so here the trunk writes into one preallocated
  ``StaticCache`` whose length counter lives on the device, the attention mask is one
  ``[2B, L_max]`` buffer (prompt mask, then ones) and nothing is read back until the end.
* A decode step then has no host-dependent control flow and fixed addresses, so it is recorded
  once as a HIP graph (trunk, head, CFG combine, draw, log-probability, next-token embedding,
  write of token and log-probability at a device-side position) and replayed ``L_img - 2`` times.
  The prompt pass and the first decode step run eagerly (the latter doubles as the warm-up a
  capture needs).
* When the trunk's projections are prepacked int4 modules, the trunk part of the step runs as
  five launches per layer over the same cache tensors (:mod:`visionrl_amd.decode_step`) instead
  of the module's some thirty tensor ops per layer; results then agree with the module path to
  bf16 roundings of the hidden states (the attention keeps fp32 probabilities), not bit for bit.
* The tail after the head is one launch (:func:`visionrl_amd.ops.cfg_sample`) when the logits are
  bf16 on a GPU, and the reference's torch formulas otherwise; both draw through
  ``exponential_`` exactly as ``torch.multinomial`` does, so a seeded rollout
  (``vrl/models/families/janus_pro/executor.py:147-151`` seeds the global generator) samples the
  same tokens as the reference loop.

The step API the executor's token scheduler drives (``init_ar_state`` / ``step_ar`` /
``finalize_ar_state``, ``policy.py:527-622``, ``executor.py:373-413``) is covered for what the
scheduler does by default: every row of the chunk stepped together at one position.  A generation
whose scheduler batch is smaller than the chunk (rows at different positions) is handed to the
policy's own step functions.
"""

from __future__ import annotations

import dataclasses
import types
import weakref
from typing import Any

import torch
import torch.nn.functional as F

from . import ops
from .decode_step import NativeDecodeTrunk, trunk_signature
from .linear import Int4Linear

__all__ = ["StaticARSampler", "StaticARState", "StaticARStepResult", "install_static_ar_sampler"]


def _round_up(n: int, to: int) -> int:
    return (n + to - 1) // to * to


@dataclasses.dataclass
class StaticARStepResult:
    """Fields of the reference's ``ARStepResult`` (``vrl/models/ar.py:26-39``)."""

    sequence_ids: list
    positions: list
    token: Any
    log_prob: Any
    replay_extras: dict = dataclasses.field(default_factory=dict)


@dataclasses.dataclass
class StaticARState:
    """What ``init_ar_state`` hands to ``step_ar`` / ``finalize_ar_state``: the rows of one chunk,
    advancing together over one static cache (the counterpart of ``JanusProARState``,
    ``policy.py:114-130``, whose per-row caches and masks have no equivalent here)."""

    session: Any
    inputs: Any                    # prompt embeddings and masks until the first step consumed them
    cfg_weight: float
    temperature: float
    image_token_num: int
    batch_size: int
    position: int = 0
    reference: Any = None          # the policy's own (init_ar_state, step_ar, finalize_ar_state), if it has them
    delegate: Any = None           # their state, once a partial batch sent the generation their way

    released: bool = False         # finalized: the session's buffers may serve another generation
    final: Any = None              # (token ids, log-probabilities) as finalize_ar_state returned them

    @property
    def finished(self) -> bool:
        return self.position >= self.image_token_num

    @property
    def token_ids(self) -> torch.Tensor:
        """Tokens sampled so far (columns from ``position`` on are not yet written).  A view of the
        session's buffer while the generation runs, a copy once it has finished: the buffer is
        rewritten by the next generation of this shape."""
        if self.released:
            return self.final[0]
        view = self.session.tokens[:, :self.image_token_num]
        return view.clone() if self.finished else view

    @property
    def logprobs(self) -> torch.Tensor:
        if self.released:
            return self.final[1]
        view = self.session.logprobs[:, :self.image_token_num]
        return view.clone() if self.finished else view


class _Session:
    """Buffers and the recorded step for one (rows, cache length, guidance, temperature) shape."""

    def __init__(self, sampler: "StaticARSampler", rows2: int, hidden: int, max_len: int,
                 dtype: torch.dtype, device: torch.device, cfg_weight: float, temperature: float,
                 mask_dtype: torch.dtype):
        from transformers.cache_utils import StaticCache

        self.sampler = sampler
        self.rows2, self.max_len = rows2, max_len
        self.cfg_weight, self.temperature = float(cfg_weight), float(temperature)
        trunk = sampler.trunk
        self.cache = StaticCache(config=trunk.config, max_cache_len=max_len)
        self.cur = torch.zeros((rows2, 1, hidden), dtype=dtype, device=device)
        self.mask = torch.ones((rows2, max_len), dtype=mask_dtype, device=device)
        self.tokens = torch.zeros((rows2 // 2, max_len), dtype=torch.long, device=device)
        self.logprobs = torch.zeros((rows2 // 2, max_len), dtype=torch.float32, device=device)
        self.img_pos = torch.zeros(1, dtype=torch.long, device=device)
        self.mask_u8 = torch.ones((rows2, max_len), dtype=torch.uint8, device=device)
        self.slot = torch.zeros(1, dtype=torch.long, device=device)   # cache slot of the next new token
        self.native = None     # NativeDecodeTrunk once the cache exists, False if the trunk does not qualify
        self.graph = None
        self.owner = None      # weak reference to the state whose generation the buffers hold
        self.head_workspace = None   # of the fused head + tail launch
        self.signature = None  # of the trunk's modules and adapter state the launch list / graph were made for

    def _head_packed(self):
        """The prepacked weight of a bare, bias-free int4 ``gen_head`` (made again first if its canonical
        buffers changed), else ``None``."""
        head = getattr(self.sampler.base, "gen_head", None)
        if isinstance(head, Int4Linear) and head.bias is None:
            return head._fresh_packed()
        return None

    # -- one call of sample_image_tokens starts here
    def begin(self, mask: torch.Tensor) -> None:
        signature = (trunk_signature(self.sampler.trunk), id(self._head_packed()))
        if signature != self.signature:   # modules swapped, adapters merged / disabled / switched: start over
            self.signature, self.native, self.graph = signature, None, None
        self.cache.reset()
        self.mask.fill_(1)
        self.mask[:, :mask.shape[1]].copy_(mask)
        self.mask_u8.copy_(self.mask != 0)
        self.slot.fill_(mask.shape[1])
        self.img_pos.zero_()

    def tail(self, hidden: torch.Tensor) -> None:
        """Head, guided draw, log-probability, bookkeeping, next input (``policy.py:684-700``)."""
        s = self.sampler
        packed = self._head_packed() if s.fused_tail and s.fused_head else None
        if packed is not None and hidden.dtype == torch.bfloat16 and hidden.is_cuda and \
                ops.head_sample_supported(self.rows2, packed):
            # head and tail in one launch: the logits never reach memory
            if self.head_workspace is None:
                self.head_workspace = ops.head_sample_workspace(self.rows2 // 2, packed.N, hidden.device)
            sampled, lp = ops.head_sample(hidden.reshape(self.rows2, -1).contiguous(), packed, self.cfg_weight, self.temperature,
                                          workspace=self.head_workspace)
            logits = None
        else:
            logits = s.base.gen_head(hidden).squeeze(1)
        if logits is None:
            pass
        elif s.fused_tail and logits.dtype == torch.bfloat16 and logits.is_cuda:
            sampled, lp = ops.cfg_sample(logits.contiguous(), self.cfg_weight, self.temperature)
        else:
            cond, uncond = logits.chunk(2, dim=0)
            guided = uncond + self.cfg_weight * (cond - uncond)
            probs = F.softmax(guided / self.temperature, dim=-1)
            sampled = torch.multinomial(probs, num_samples=1).squeeze(-1)
            lp = F.log_softmax(cond / self.temperature, dim=-1).gather(-1, sampled.unsqueeze(-1)).squeeze(-1)
        self.tokens.index_copy_(1, self.img_pos, sampled.unsqueeze(1))
        self.logprobs.index_copy_(1, self.img_pos, lp.to(torch.float32).unsqueeze(1))
        self.img_pos.add_(1)
        nxt = s.base.prepare_gen_img_embeds(torch.cat([sampled, sampled], dim=0).unsqueeze(-1))
        self.cur.copy_(nxt.reshape(self.cur.shape))

    def prefill(self, embeds: torch.Tensor) -> None:
        out = self.sampler.trunk(inputs_embeds=embeds, attention_mask=self.mask, use_cache=True,
                                 past_key_values=self.cache)
        self.tail(out.last_hidden_state[:, -1:, :])
        if self.native is None:   # the cache tensors exist from here on
            self.native = False
            s = self.sampler
            if s.native and self.cur.is_cuda and self.cur.dtype == torch.bfloat16 and \
                    NativeDecodeTrunk.unsupported(s.trunk, self.rows2, self.max_len) is None:
                try:
                    self.native = NativeDecodeTrunk(s.trunk, self.cache, self.cur, self.mask_u8, self.slot)
                except (TypeError, ValueError):   # something the native launches do not take: module path
                    self.native = False

    def step(self) -> None:
        if self.native:
            hidden = self.native.run().view(self.rows2, 1, -1)
        else:
            out = self.sampler.trunk(inputs_embeds=self.cur, attention_mask=self.mask, use_cache=True,
                                     past_key_values=self.cache)
            hidden = out.last_hidden_state[:, -1:, :]
        self.tail(hidden)
        self.slot.add_(1)

    def capture(self) -> None:
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            self.step()
        self.graph = graph


class StaticARSampler:
    """``sample_image_tokens`` of a Janus-Pro style policy over a static cache and a HIP graph.

    ``policy`` is duck-typed: ``_lm_trunk()`` returns the Hugging Face ``LlamaModel``
    (``policy.py:240-266``), ``_base()`` the module holding ``gen_head`` and
    ``prepare_gen_img_embeds`` (``policy.py:226-238``), ``config`` the defaults
    (``cfg_weight``, ``temperature``, ``image_token_num``).  ``graph=False`` runs every step
    eagerly (same arithmetic, same random stream); ``fused_tail=False`` keeps the torch formulas
    for the part after the head; ``fused_head=False`` keeps the head a launch of its own in front of
    the fused tail (with it, a prepacked int4 ``gen_head`` and the tail are one launch and the logits
    are never written).  With ``native`` (the default) the trunk of a decode step runs as
    :class:`visionrl_amd.decode_step.NativeDecodeTrunk` (five launches per layer, six with LoRA
    adapters on the attention projections) when the policy went through ``apply_int4_to_policy``
    with its defaults; otherwise, and for the prompt pass, the trunk module itself is called.
    """

    def __init__(self, policy: Any, *, graph: bool = True, fused_tail: bool = True, native: bool = True,
                 fused_head: bool = True, length_bucket: int = 64, max_sessions: int = 2):
        self.policy = policy
        self.trunk = policy._lm_trunk()
        self.base = policy._base()
        for name in ("gen_head", "prepare_gen_img_embeds"):
            if not hasattr(self.base, name):
                raise TypeError(f"policy._base() has no {name}")
        self.graph = bool(graph)
        self.fused_tail = bool(fused_tail)
        self.fused_head = bool(fused_head)
        self.native = bool(native)
        self.length_bucket = int(length_bucket)
        self.max_sessions = int(max_sessions)
        self._sessions: dict = {}

    def _defaults(self, cfg_weight, temperature, image_token_num):
        conf = getattr(self.policy, "config", None)
        cfg = cfg_weight if cfg_weight is not None else getattr(conf, "cfg_weight", None)
        temp = temperature if temperature is not None else getattr(conf, "temperature", None)
        n_img = image_token_num or getattr(conf, "image_token_num", None)
        if cfg is None or temp is None or not n_img:
            raise ValueError("cfg_weight, temperature and image_token_num need a value or a policy.config default")
        if not float(temp) > 0:
            raise ValueError("temperature must be positive")
        return float(cfg), float(temp), int(n_img)

    def _session(self, key, make):
        """The cached session of this shape if no live generation holds it, else a new one (which
        takes its place in the cache; the busy one stays with its state until that is finalized or
        dropped).  The reference's states are independent objects (``policy.py:114-130``); here two
        states of one shape must not share cache, token and log-probability buffers."""
        sess = self._sessions.pop(key, None)
        if sess is not None and sess.owner is not None:
            holder = sess.owner()
            if holder is not None and not holder.released:
                sess = None
        if sess is None:
            while len(self._sessions) >= self.max_sessions:   # oldest first: caches are GBs at 1B scale
                self._sessions.pop(next(iter(self._sessions)))
            sess = make()
        self._sessions[key] = sess
        return sess

    # -- the step API (init_ar_state / step_ar / finalize_ar_state, policy.py:527-622) ---------------
    @torch.no_grad()
    def init_ar_state(self, cond_inputs_embeds: torch.Tensor, uncond_inputs_embeds: torch.Tensor,
                      cond_attention_mask: torch.Tensor, uncond_attention_mask: torch.Tensor, *,
                      cfg_weight: float | None = None, temperature: float | None = None,
                      image_token_num: int | None = None) -> "StaticARState":
        """State for a generation whose rows advance together; nothing runs until the first step."""
        cfg, temp, n_img = self._defaults(cfg_weight, temperature, image_token_num)
        if cond_inputs_embeds.dim() != 3 or cond_inputs_embeds.shape != uncond_inputs_embeds.shape:
            raise ValueError("cond and uncond embeddings must both be [B, L_text, H]")
        B, n_text, hidden = cond_inputs_embeds.shape
        if tuple(cond_attention_mask.shape) != (B, n_text) or tuple(uncond_attention_mask.shape) != (B, n_text):
            raise ValueError("attention masks must be [B, L_text]")
        device, dtype = cond_inputs_embeds.device, cond_inputs_embeds.dtype
        max_len = _round_up(n_text + n_img, self.length_bucket)
        key = (2 * B, hidden, max_len, dtype, device, cfg, temp, cond_attention_mask.dtype)
        sess = self._session(key, lambda: _Session(self, 2 * B, hidden, max_len, dtype, device, cfg, temp,
                                                   cond_attention_mask.dtype))
        state = StaticARState(session=sess, inputs=(cond_inputs_embeds, uncond_inputs_embeds, cond_attention_mask,
                                                    uncond_attention_mask),
                              cfg_weight=cfg, temperature=temp, image_token_num=n_img, batch_size=B)
        sess.owner = weakref.ref(state)
        return state

    def _advance(self, state: "StaticARState") -> None:
        """One token for every row: the prompt pass first, then eager / recorded decode steps."""
        sess = state.session
        if state.released:
            raise ValueError("the state was finalized")
        if state.position >= state.image_token_num:
            raise ValueError("the generation has already finished sampling")
        if state.position == 0:
            cond, uncond, cmask, umask = state.inputs
            sess.begin(torch.cat([cmask, umask], dim=0))
            sess.prefill(torch.cat([cond, uncond], dim=0))
            state.inputs = None
        elif self.graph and sess.cur.is_cuda:
            if sess.graph is None and state.position >= 2:
                sess.capture()           # after one eager decode step: records, does not run
            if sess.graph is None:
                sess.step()              # a real step, and the warm-up the capture needs
            else:
                sess.graph.replay()
        else:
            sess.step()
        state.position += 1

    @torch.no_grad()
    def step_ar(self, state: "StaticARState", sequences, *, generator=None) -> "StaticARStepResult":
        """One scheduled token step (``JanusProPolicy.step_ar``, ``policy.py:527-572``) for all rows at once.

        ``sequences`` are the scheduler's active sequences (``metadata["row_index"]``, ``position``,
        ``sample_id``).  The token scheduler hands over every row of a chunk at one position unless
        it was given a smaller batch size (``executor.py:396-413``); a partial batch on the first
        step switches the whole generation to the policy's own step functions, later it is an error.
        """
        del generator   # like the reference: the draw uses the global generator
        if not sequences:
            raise ValueError("step_ar requires at least one ActiveSequence")
        if state.delegate is not None:
            return state.reference[1](state.delegate, sequences)
        B = state.batch_size
        rows = [int(seq.metadata.get("row_index", -1)) for seq in sequences]
        if any(row < 0 or row >= B for row in rows):
            raise ValueError(f"invalid Janus row indices: {rows}")
        positions = [int(seq.position) for seq in sequences]
        if len(set(positions)) != 1:
            raise ValueError("ActiveSequence positions must match within one AR step")
        if rows != list(range(B)):
            if state.position == 0 and state.reference is not None:
                cond, uncond, cmask, umask = state.inputs
                state.delegate = state.reference[0](cond, uncond, cmask, umask, cfg_weight=state.cfg_weight,
                                                    temperature=state.temperature,
                                                    image_token_num=state.image_token_num)
                return state.reference[1](state.delegate, sequences)
            raise ValueError("the static decode loop steps all rows of a chunk together, in row order; "
                             f"got rows {rows} of {B}")
        if positions[0] != state.position:
            raise ValueError("ActiveSequence positions must match the state's position")
        p = state.position
        self._advance(state)
        sess = state.session
        return StaticARStepResult(sequence_ids=[str(seq.sample_id) for seq in sequences], positions=positions,
                                  token=sess.tokens[:, p].clone(), log_prob=sess.logprobs[:, p].clone())

    @torch.no_grad()
    def finalize_ar_state(self, state: "StaticARState") -> tuple[torch.Tensor, torch.Tensor]:
        """``(image_token_ids, logprobs)`` of the rows sampled so far up to ``image_token_num``."""
        if state.delegate is not None:
            return state.reference[2](state.delegate)
        if state.released:
            raise ValueError("the state was finalized before")
        n = state.image_token_num
        out = state.session.tokens[:, :n].clone(), state.session.logprobs[:, :n].clone()
        state.final, state.released = out, True    # the session may serve the next generation of this shape
        return out

    @torch.no_grad()
    def sample_image_tokens(self, cond_inputs_embeds: torch.Tensor, uncond_inputs_embeds: torch.Tensor,
                            cond_attention_mask: torch.Tensor, uncond_attention_mask: torch.Tensor, *,
                            cfg_weight: float | None = None, temperature: float | None = None,
                            image_token_num: int | None = None) -> tuple[torch.Tensor, torch.Tensor]:
        """Returns ``(image_token_ids int64 [B, L_img], logprobs float32 [B, L_img])``."""
        state = self.init_ar_state(cond_inputs_embeds, uncond_inputs_embeds, cond_attention_mask,
                                   uncond_attention_mask, cfg_weight=cfg_weight, temperature=temperature,
                                   image_token_num=image_token_num)
        while state.position < state.image_token_num:
            self._advance(state)
        return self.finalize_ar_state(state)


def install_static_ar_sampler(policy: Any, **options) -> StaticARSampler:
    """Route ``policy.sample_image_tokens`` (what ``JanusProPipelineExecutor.forward`` calls,
    ``vrl/models/families/janus_pro/executor.py:197-203``) and the step API the executor's token
    scheduler drives (``init_ar_state`` / ``step_ar`` / ``finalize_ar_state``, ``executor.py:373-413``)
    through a :class:`StaticARSampler`.  The policy's own step functions, if it has them, stay
    reachable: a generation whose first scheduled batch is not the whole chunk is handed to them."""
    sampler = StaticARSampler(policy, **options)
    names = ("init_ar_state", "step_ar", "finalize_ar_state")
    reference = tuple(getattr(policy, name, None) for name in names)
    reference = reference if all(callable(fn) for fn in reference) else None

    def sample_image_tokens(self, cond_inputs_embeds, uncond_inputs_embeds, cond_attention_mask,
                            uncond_attention_mask, *, cfg_weight=None, temperature=None, image_token_num=None):
        return sampler.sample_image_tokens(cond_inputs_embeds, uncond_inputs_embeds, cond_attention_mask,
                                           uncond_attention_mask, cfg_weight=cfg_weight,
                                           temperature=temperature, image_token_num=image_token_num)

    def init_ar_state(self, cond_inputs_embeds, uncond_inputs_embeds, cond_attention_mask, uncond_attention_mask, *,
                      cfg_weight=None, temperature=None, image_token_num=None):
        state = sampler.init_ar_state(cond_inputs_embeds, uncond_inputs_embeds, cond_attention_mask,
                                      uncond_attention_mask, cfg_weight=cfg_weight, temperature=temperature,
                                      image_token_num=image_token_num)
        state.reference = reference
        return state

    def step_ar(self, state, sequences, *, generator=None):
        return sampler.step_ar(state, sequences, generator=generator)

    def finalize_ar_state(self, state):
        return sampler.finalize_ar_state(state)

    policy.sample_image_tokens = types.MethodType(sample_image_tokens, policy)
    policy.init_ar_state = types.MethodType(init_ar_state, policy)
    policy.step_ar = types.MethodType(step_ar, policy)
    policy.finalize_ar_state = types.MethodType(finalize_ar_state, policy)
    policy._static_ar_sampler = sampler
    return sampler
