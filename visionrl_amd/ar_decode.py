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
import gc
import types
import weakref
from typing import Any

import torch
import torch.nn.functional as F

from torch import nn

from . import ops
from .decode_step import NativeDecodeTrunk, trunk_signature
from .linear import Int4Linear, _source_changed, _source_state

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
    row_positions: Any = None      # per-row positions once the scheduler stepped a part of the rows (else None)

    @property
    def finished(self) -> bool:
        if self.row_positions is not None:
            return min(self.row_positions) >= self.image_token_num
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

        self._sampler = weakref.ref(sampler)   # no cycle with the sampler's table of sessions: a dropped sampler frees
                                               # its sessions (recorded graphs included) at once, not in some later
                                               # garbage collection that may fall into another session's recording
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
        self.graph_short = None   # the step with the launch list for a cache that is still short, where there is one
        self.eager_steps = [0, 0]  # eager decode steps so far with the default / the short list (a recording's warm-up)
        self.prompt_len = 0        # slots the prompt pass filled
        self.owner = None      # weak reference to the state whose generation the buffers hold
        self.head_workspace = None   # of the fused head + tail launch
        self.signature = None  # of the trunk's modules and adapter state the launch list / graph were made for
        self.head_verified = None    # the signature under which the head's split into (front, last linear) was checked
        self.front_call = None       # the front of a two-layer head as one launch over the native trunk's output
        self.sampled = torch.zeros(rows2 // 2, dtype=torch.long, device=device)
        self.lp = torch.zeros(rows2 // 2, dtype=torch.float32, device=device)

    def _head_parts(self):
        """``(front modules, last linear)`` when ``gen_head`` is an int4 linear, an ``nn.Sequential`` that ends
        in one, or a module shaped like the checkpoints' ``vision_head`` (``output_mlp_projector``,
        ``vision_activation``, ``vision_head``, applied in that order: Linear, GELU, Linear); else ``None``."""
        head = getattr(self.sampler.base, "gen_head", None)
        if isinstance(head, Int4Linear):
            return [], head
        if isinstance(head, nn.Sequential) and len(head) >= 1 and isinstance(head[-1], Int4Linear):
            return list(head)[:-1], head[-1]
        names = ("output_mlp_projector", "vision_activation", "vision_head")
        if all(isinstance(getattr(head, n, None), nn.Module) for n in names) and \
                isinstance(head.vision_head, Int4Linear):
            return [head.output_mlp_projector, head.vision_activation], head.vision_head
        return None

    def _head_packed(self):
        """The prepacked weight of the head's last int4 linear (made again first if its canonical buffers
        changed), else ``None``."""
        parts = self._head_parts()
        return parts[1]._fresh_packed() if parts is not None else None

    def _front_packed(self):
        """The prepacked weight of the front of a two-layer head when that front is an int4 linear followed by
        an exact GELU (one launch with the epilogue), else ``None``."""
        parts = self._head_parts()
        if parts is None or len(parts[0]) != 2:
            return None
        lin, act = parts[0]
        if isinstance(lin, Int4Linear) and isinstance(act, nn.GELU) and getattr(act, "approximate", "none") == "none":
            return lin._fresh_packed()
        return None

    # -- one call of sample_image_tokens starts here
    def begin(self, mask: torch.Tensor) -> None:
        signature = (trunk_signature(self.sampler.trunk), id(self._head_packed()), id(self._front_packed()))
        if signature != self.signature:   # modules swapped, adapters merged / disabled / switched: start over
            self.signature, self.native, self.graph, self.graph_short = signature, None, None, None
            self.eager_steps = [0, 0]
            self.head_workspace = None    # sized for the head it was made for
            self.front_call = None
        self.cache.reset()
        self.mask.fill_(1)
        self.mask[:, :mask.shape[1]].copy_(mask)
        self.mask_u8.copy_(self.mask != 0)
        self.slot.fill_(mask.shape[1])
        self.prompt_len = int(mask.shape[1])
        self.img_pos.zero_()

    def _front(self, parts, hidden: torch.Tensor) -> torch.Tensor:
        """The modules of the head in front of its last linear, applied to ``[rows, 1, hidden]``."""
        for module in parts[0]:
            hidden = module(hidden)
        return hidden

    def _head_split_ok(self, parts, hidden: torch.Tensor) -> bool:
        """Whether the head's last linear over its front is the head: checked once per set of modules, eagerly, on
        the prompt pass's hidden state (an unknown ``forward`` could do more than the three attributes say)."""
        if not parts[0] or self.head_verified == self.signature:
            return True
        if torch.cuda.is_current_stream_capturing():
            return False
        same = torch.equal(self.sampler.base.gen_head(hidden), parts[1](self._front(parts, hidden)))
        if same:
            self.head_verified = self.signature
        return same

    def tail(self, hidden, advance_slot: bool = False) -> None:
        """Head, guided draw, log-probability, bookkeeping, next input (``policy.py:684-700``).  ``hidden`` is
        the trunk's ``[rows, 1, hidden]`` output, or ``None`` when the native trunk left its last norm to the
        head's front launch.  ``advance_slot``: a decode step, after which the cache slot moves on."""
        s = self.sampler
        parts = self._head_parts() if s.fused_tail and s.fused_head else None
        packed = parts[1]._fresh_packed() if parts is not None else None
        fused = packed is not None and self.cur.dtype == torch.bfloat16 and self.cur.is_cuda and \
            ops.head_sample_supported(self.rows2, packed) and (hidden is None or self._head_split_ok(parts, hidden))
        if hidden is None and not fused:
            raise RuntimeError("the trunk left its last norm to a head launch that does not exist")
        if fused:
            # head and tail in one call: the logits never reach memory, and the call writes token and
            # log-probability at the position, moves the counters on and looks the next input up
            if hidden is None:
                rows = self.front_call.launch()
            elif parts[0] and self.front_call is not None and self.native and self.native.normed is not None and \
                    hidden.data_ptr() == self.native.normed.data_ptr():
                rows = self.front_call.launch()
            else:
                rows = self._front(parts, hidden).reshape(self.rows2, -1).contiguous()
            if self.head_workspace is None:
                self.head_workspace = ops.head_sample_workspace(self.rows2 // 2, packed.N, rows.device)
            table = s.embedding_table(packed.N, self.cur)
            ops.head_sample(rows, packed, self.cfg_weight, self.temperature, workspace=self.head_workspace,
                            out=(self.sampled, self.lp), bias=parts[1].bias,
                            bookkeeping=(self.tokens, self.logprobs, self.img_pos, self.slot if advance_slot else None),
                            embedding=None if table is None else (table, self.cur))
            if table is None:
                nxt = s.base.prepare_gen_img_embeds(torch.cat([self.sampled, self.sampled], dim=0).unsqueeze(-1))
                self.cur.copy_(nxt.reshape(self.cur.shape))
            return
        logits = s.base.gen_head(hidden).squeeze(1)
        if s.fused_tail and logits.dtype == torch.bfloat16 and logits.is_cuda:
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
        if advance_slot:
            self.slot.add_(1)

    def prefill(self, embeds: torch.Tensor) -> None:
        out = self.sampler.trunk(inputs_embeds=embeds, attention_mask=self.mask, use_cache=True,
                                 past_key_values=self.cache)
        self.tail(out.last_hidden_state[:, -1:, :])
        if self.native is None:   # the cache tensors exist from here on
            self.native = False
            s = self.sampler
            if s.native and self.cur.is_cuda and self.cur.dtype == torch.bfloat16 and \
                    NativeDecodeTrunk.unsupported(s.trunk, self.rows2, self.max_len) is None:
                # a two-layer head whose front is one launch takes the trunk's last norm along
                front = self._front_packed() if s.fused_tail and s.fused_head and \
                    self.head_verified == self.signature and \
                    ops.head_sample_supported(self.rows2, self._head_packed()) else None
                try:
                    self.native = NativeDecodeTrunk(s.trunk, self.cache, self.cur, self.mask_u8, self.slot,
                                                    final_norm=front is None)
                    if front is not None:
                        bias = self._head_parts()[0][0].bias
                        if self.native.final is not None:
                            x, res, w, eps = self.native.final
                            self.front_call = ops.EpilogueGemv(x, front, bias, gelu=True, norm=(res, w, eps))
                        else:
                            self.front_call = ops.EpilogueGemv(self.native.normed, front, bias, gelu=True)
                except (TypeError, ValueError):   # something the native launches do not take: module path
                    self.native, self.front_call = False, None

    # -- rows that advance at different times (the scheduler's partial batches) -------------------------
    def rows_mode_supported(self) -> bool:
        """Whether a part of the rows can be stepped over the static cache: the native trunk and the one-call
        head (the module trunk shares one cache position between the rows of a call)."""
        s = self.sampler
        packed = self._head_packed() if s.fused_tail and s.fused_head else None
        return bool(s.native and self.cur.is_cuda and self.cur.dtype == torch.bfloat16 and packed is not None and
                    ops.head_sample_supported(self.rows2, packed) and
                    NativeDecodeTrunk.unsupported(s.trunk, self.rows2, self.max_len) is None)

    def enter_rows_mode(self, prompt_len: int, position: int) -> None:
        """Counters per row (cache slot of the 2B rows, image position of the B pairs) in place of the shared
        ones, all at ``position``; the launch list over them is made with the first decode step."""
        B, dev = self.rows2 // 2, self.cur.device
        self.slot_rows = torch.full((self.rows2,), prompt_len + max(position - 1, 0), dtype=torch.long, device=dev)
        self.pos_rows = torch.full((B,), position, dtype=torch.long, device=dev)
        self.active = torch.zeros(B, dtype=torch.uint8, device=dev)
        self.noise_rows = None
        self.native_rows = None
        self.prompt_hidden = None

    def prefill_rows(self, embeds: torch.Tensor) -> None:
        """The prompt pass of every row at once; nothing is drawn yet (a row's first token is drawn when the
        scheduler steps it, so the random stream is used in the order of the reference's per-row loop)."""
        out = self.sampler.trunk(inputs_embeds=embeds, attention_mask=self.mask, use_cache=True,
                                 past_key_values=self.cache)
        self.prompt_hidden = out.last_hidden_state[:, -1:, :].clone()

    def step_rows(self, rows: list, first: bool) -> None:
        """One token for the pairs ``rows``: the trunk runs over every row (a row outside the batch repeats its
        last step into the same cache slot, which changes nothing), the head's call writes, counts and
        embeds for the rows of the batch only."""
        s = self.sampler
        B = self.rows2 // 2
        if first:
            hidden = self.prompt_hidden
        else:
            if self.native_rows is None:
                self.native_rows = NativeDecodeTrunk(s.trunk, self.cache, self.cur, self.mask_u8, self.slot_rows)
            hidden = self.native_rows.run().view(self.rows2, 1, -1)
        parts = self._head_parts()
        packed = parts[1]._fresh_packed()
        if parts[0] and not self._head_split_ok(parts, hidden):
            raise RuntimeError("gen_head is not its last linear over its front modules")
        front = self._front(parts, hidden).reshape(self.rows2, -1).contiguous()
        idx = torch.tensor(rows, dtype=torch.long, device=self.cur.device)
        self.active.zero_()
        self.active[idx] = 1
        # the draws of the batch, in its order, as torch.multinomial would make them for these rows alone
        if self.noise_rows is None:
            self.noise_rows = torch.ones((B, packed.N), dtype=torch.bfloat16, device=self.cur.device)
        self.noise_rows[idx] = torch.empty((len(rows), packed.N), dtype=torch.bfloat16,
                                           device=self.cur.device).exponential_(1.0)
        if self.head_workspace is None:
            self.head_workspace = ops.head_sample_workspace(B, packed.N, front.device)
        table = s.embedding_table(packed.N, self.cur)
        ops.head_sample(front, packed, self.cfg_weight, self.temperature, workspace=self.head_workspace,
                        noise=self.noise_rows, out=(self.sampled, self.lp), bias=parts[1].bias,
                        bookkeeping=(self.tokens, self.logprobs, self.pos_rows, None if first else self.slot_rows),
                        embedding=None if table is None else (table, self.cur), per_row=True, active=self.active)
        if table is None:
            picked = self.sampled[idx]
            nxt = s.base.prepare_gen_img_embeds(torch.cat([picked, picked], dim=0).unsqueeze(-1))
            self.cur[torch.cat([idx, idx + B])] = nxt.reshape(2 * len(rows), 1, -1)

    def short_form(self, position: int) -> bool:
        """Whether the decode step that samples image token ``position`` (>= 1) takes the native trunk's launch
        list for a short cache: the slots filled by then are the prompt's and one per earlier step."""
        return bool(self.native) and self.native.short_form(self.prompt_len + position - 1)

    def step(self, short: bool = False) -> None:
        if self.native:
            hidden = self.native.run(short)
            hidden = hidden.view(self.rows2, 1, -1) if hidden is not None else None
        else:
            out = self.sampler.trunk(inputs_embeds=self.cur, attention_mask=self.mask, use_cache=True,
                                     past_key_values=self.cache)
            hidden = out.last_hidden_state[:, -1:, :]
        self.tail(hidden, advance_slot=True)

    @property
    def sampler(self) -> "StaticARSampler":
        sampler = self._sampler()
        if sampler is None:
            raise RuntimeError("the sampler this session belongs to no longer exists")
        return sampler

    def capture(self, short: bool = False) -> None:
        graph = torch.cuda.CUDAGraph()
        # No cyclic garbage collection while the stream records: a finalizer that releases device resources (another
        # recorded graph, say) in the middle of a recording ends the process.  torch.cuda.graph collects once itself
        # before the recording begins.
        collecting = gc.isenabled()
        gc.disable()
        try:
            with torch.cuda.graph(graph):
                self.step(short)
        finally:
            if collecting:
                gc.enable()
        if short:
            self.graph_short = graph
        else:
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
    are never written; a two-layer head runs its front as one launch with bias and GELU and its last linear
    in that call); ``embed_table`` see :meth:`embedding_table`.  With ``native`` (the default) the trunk of a decode step runs as
    :class:`visionrl_amd.decode_step.NativeDecodeTrunk` (five launches per layer, six with LoRA
    adapters on the attention projections) when the policy went through ``apply_int4_to_policy``
    with its defaults; otherwise, and for the prompt pass, the trunk module itself is called.
    """

    def __init__(self, policy: Any, *, graph: bool = True, fused_tail: bool = True, native: bool = True,
                 fused_head: bool = True, embed_table: "bool | str" = "auto", length_bucket: int = 64,
                 max_sessions: int = 2):
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
        if embed_table not in (True, False, "auto"):
            raise ValueError('embed_table is True, False or "auto"')
        self.embed_table = embed_table
        self._table = None          # (tensor, state of the parameters it was made from) once built
        self._table_refused = None  # the parameter state under which tabulating was tried and dropped
        self.length_bucket = int(length_bucket)
        self.max_sessions = int(max_sessions)
        self._sessions: dict = {}

    def _embedding_params(self):
        """The parameters ``prepare_gen_img_embeds`` reads in the checkpoints' layout (``gen_embed``, then
        ``gen_aligner``; ``policy.py:698-700`` calls it), or ``None`` when the base holds neither."""
        mods = [m for m in (getattr(self.base, n, None) for n in ("gen_embed", "gen_aligner")) if isinstance(m, nn.Module)]
        if not mods:
            return None
        return [p for m in mods for p in list(m.parameters()) + list(m.buffers())]

    def embedding_table(self, V: int, cur: torch.Tensor):
        """``prepare_gen_img_embeds`` tabulated over the ``V`` image tokens (bf16 ``[V, hidden]``: the next input
        is a function of the sampled token alone), for the head launch to look the next input up itself; ``None``
        where that is switched off or would not be the module's own result.

        ``"auto"``: built when the base holds ``gen_embed`` / ``gen_aligner`` (their parameters' modification
        counters say when to build it again, in place) and a handful of tokens evaluated at the step's own batch
        size give the tabulated rows bit for bit (a GEMM library may round a 16384-row product differently
        from a two-row one: then the modules keep running every step).  ``True`` skips both conditions."""
        if self.embed_table is False or not cur.is_cuda or cur.dtype != torch.bfloat16:
            return None
        params = self._embedding_params()
        if params is None and self.embed_table != True:   # noqa: E712 ("auto" is truthy)
            return None
        if self._table is not None and (params is None or not _source_changed(self._table[1], *params)) and \
                self._table[0].shape[0] == V:
            return self._table[0]
        if self._table_refused is not None and params is not None and \
                not _source_changed(self._table_refused, *params):
            return None
        if torch.cuda.is_current_stream_capturing():
            return self._table[0] if self._table is not None else None
        ids = torch.arange(V, device=cur.device)
        try:
            table = self.base.prepare_gen_img_embeds(ids.unsqueeze(-1)).reshape(V, -1)
        except (RuntimeError, IndexError):   # the embedding holds fewer tokens than the head
            table = None
        rows2 = cur.shape[0]
        ok = table is not None and table.dtype == torch.bfloat16 and table.shape[1] == cur.shape[-1] and \
            table.shape[1] % 8 == 0
        if ok and self.embed_table == "auto":
            probe = (torch.arange(rows2, device=cur.device) * 2654435761 + 12345) % V
            probe[0], probe[-1] = 0, V - 1
            ok = torch.equal(self.base.prepare_gen_img_embeds(probe.unsqueeze(-1)).reshape(rows2, -1), table[probe])
        state = _source_state(*params) if params is not None else ()
        if not ok:
            self._table, self._table_refused = None, state
            return None
        if self._table is not None and self._table[0].shape == table.shape:
            self._table[0].copy_(table)      # in place: recorded steps hold its address
            self._table = (self._table[0], state)
        else:
            self._table = (table.contiguous(), state)
        return self._table[0]

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
            # two recordings where the native trunk has a launch list of its own for a short cache: the
            # step is replayed from the one that fits the slots filled so far
            short = sess.short_form(state.position)
            graph = sess.graph_short if short else sess.graph
            if graph is None and sess.eager_steps[short] >= 1:
                sess.capture(short)      # after one eager decode step of that form: records, does not run
                graph = sess.graph_short if short else sess.graph
            if graph is None:
                sess.step(short)         # a real step, and the warm-up the capture needs
                sess.eager_steps[short] += 1
            else:
                graph.replay()
        else:
            sess.step(sess.short_form(state.position))
        state.position += 1

    def _advance_rows(self, state: "StaticARState", rows: list, position: int, sequences) -> "StaticARStepResult":
        """One token for a part of the rows (``JanusProPolicy._sample_ar_step`` with ``row_indices``,
        ``policy.py:624-731``), over the static cache with one slot counter per row."""
        sess = state.session
        if state.released:
            raise ValueError("the state was finalized")
        if len(set(rows)) != len(rows):
            raise ValueError(f"duplicate Janus row indices: {rows}")
        if state.row_positions is None:          # the first partial batch: counters per row from here on
            if state.position == 0:
                cond, uncond, cmask, umask = state.inputs
                sess.begin(torch.cat([cmask, umask], dim=0))
                sess.enter_rows_mode(cmask.shape[1], 0)
                sess.prefill_rows(torch.cat([cond, uncond], dim=0))
                state.inputs = None
            else:
                sess.enter_rows_mode(int(sess.slot.item()) - (state.position - 1), state.position)
            state.row_positions = [state.position] * state.batch_size
        if any(state.row_positions[row] != position for row in rows):
            raise ValueError("requested position does not match row positions")
        if position >= state.image_token_num:
            raise ValueError("the generation has already finished sampling")
        sess.step_rows(rows, first=position == 0)
        for row in rows:
            state.row_positions[row] += 1
        state.position = min(state.row_positions)
        idx = torch.tensor(rows, dtype=torch.long, device=sess.tokens.device)
        return StaticARStepResult(sequence_ids=[str(seq.sample_id) for seq in sequences],
                                  positions=[position] * len(rows),
                                  token=sess.tokens[idx, position], log_prob=sess.logprobs[idx, position])

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
        if rows != list(range(B)) or state.row_positions is not None:
            if state.row_positions is None and not state.session.rows_mode_supported():
                if state.position == 0 and state.reference is not None:
                    cond, uncond, cmask, umask = state.inputs
                    state.delegate = state.reference[0](cond, uncond, cmask, umask, cfg_weight=state.cfg_weight,
                                                        temperature=state.temperature,
                                                        image_token_num=state.image_token_num)
                    return state.reference[1](state.delegate, sequences)
                raise ValueError("this policy's static decode loop steps all rows of a chunk together, in row "
                                 f"order; got rows {rows} of {B}")
            return self._advance_rows(state, rows, positions[0], sequences)
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
            return state.final     # like the reference's (``policy.py:616-622``), a second call returns the same
        n = state.image_token_num
        out = state.session.tokens[:, :n].clone(), state.session.logprobs[:, :n].clone()
        if state.finished:         # the session may serve the next generation of this shape
            state.final, state.released = out, True
        return out                 # of an unfinished generation: a copy, and stepping stays legal

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
