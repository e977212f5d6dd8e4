"""The engine loop and the Python entry point.

Same surface as the reference's ``LLMEngine`` (clockwork/engine/llm_engine.py:35-242):
``add_request``, ``step``, ``generate``, ``abort_request``, ``has_unfinished_requests``,
``stats``. A tokenizer is optional here: token ids in, token ids out is the primary
mode; text (prompts, stop strings, ``RequestOutput.text``) needs a tokenizer with
``encode``/``decode``.
"""

from __future__ import annotations

import itertools
from typing import Optional

import numpy as np
import torch

from clockwork_amd.cache.prefix import PrefixCache
from clockwork_amd.config.engine import EngineConfig
from clockwork_amd.engine.batch import StepEntry
from clockwork_amd.engine.model_runner import GRAPH_BATCH_SIZES, ModelRunner
from clockwork_amd.engine.scheduler import Scheduler
from clockwork_amd.engine.sequence import RequestOutput, SamplingParams, Sequence, SequenceStatus
from clockwork_amd.sampling.sampler import Sampler


class _RequestText:
    """The text a request has produced so far, grown token by token.

    A token's text can depend on the tokens around it (a character spread over several tokens,
    a leading space that depends on what came before), so new text is never decoded from the
    new token alone: the tokens from ``anchor`` on are decoded with and without the newcomers
    and the difference is what they added (clockwork/engine/llm_engine.py:187-198). While the
    decoded tail ends in U+FFFD a character is still incomplete and nothing is shown."""

    __slots__ = ("shown", "anchor", "rendered")

    def __init__(self) -> None:
        self.shown = ""      # text handed out so far (cut where a stop string began)
        self.anchor = 0      # first output token of the decoding window
        self.rendered = 0    # output tokens whose text has been handed out

    def grow(self, decode, output_ids: list) -> str:
        """Text that the tokens past ``rendered`` add; "" while they end inside a character."""
        with_new = decode(output_ids[self.anchor:])
        if with_new.endswith("\ufffd"):
            return ""
        known = decode(output_ids[self.anchor:self.rendered])
        self.anchor, self.rendered = self.rendered, len(output_ids)
        return with_new[len(known):]

    def accept(self, addition: str, stop_strings) -> tuple[str, bool]:
        """Append ``addition``, unless a stop string shows up: then the text ends where the
        earliest one begins (llm_engine.py:211-221). Returns (what was really added, stopped)."""
        text = self.shown + addition
        starts = [at for at in map(text.find, stop_strings) if at >= 0]
        if starts:
            text = text[: min(starts)]
        added = text[len(self.shown):]  # nothing if the stop string began in text already shown
        self.shown = text
        return added, bool(starts)


class LLMEngine:
    def __init__(self, cfg: EngineConfig, tokenizer=None, runner: Optional[ModelRunner] = None,
                 weight_source=None, config_dict: Optional[dict] = None) -> None:
        self.cfg = cfg
        self.runner = runner if runner is not None else ModelRunner(
            cfg, weight_source=weight_source, config_dict=config_dict
        )
        self.tokenizer = tokenizer
        self.manager = self.runner.manager
        if cfg.model.tune_products:
            chunk = cfg.scheduler.max_num_batched_tokens
            if cfg.scheduler.max_prefill_chunk > 0:
                chunk = min(chunk, cfg.scheduler.max_prefill_chunk)
            self.runner.tune_products([chunk, *GRAPH_BATCH_SIZES])
        self.prefix_cache = PrefixCache(
            cfg.cache.block_size,
            share=self.manager.share_handle,
            drop=self.manager.drop_handle,
            enabled=cfg.cache.enable_prefix_cache and self.manager.supports_prefix_sharing,
            share_many=self.manager.share_handles,
        )
        self.scheduler = Scheduler(cfg.scheduler, self.manager, self.prefix_cache)
        self.sampler = Sampler(self.runner.device, cfg.model.seed)
        self._eos_ids = self._resolve_eos()
        self._seqs: dict[str, Sequence] = {}
        self._text: dict[str, _RequestText] = {}
        # arrival "times" are a counter, so order never depends on the clock (llm_engine.py:57-59)
        self._arrivals = itertools.count()
        self._generate_ids = itertools.count()
        self._ahead = None          # (SchedulerOutput, runner handle) made one step ahead
        self._started = None        # (SchedulerOutput, sampled tokens on the device, their copy) of a step on the GPU
        # sampled tokens come to the host through two pinned buffers, in turn: the copy of one
        # step's tokens can be under way while the step before it is still being read
        width = max(cfg.scheduler.max_num_seqs, GRAPH_BATCH_SIZES[-1], 1)
        self._token_bufs = [torch.empty(width, dtype=torch.int32, pin_memory=True) for _ in range(2)]
        self._token_buf_at = 0
        self.lookahead_steps = 0    # steps that ran from such a schedule

    def _look_ahead(self, out):
        """(schedule, runner handle) of the step after ``out`` if it can be decided before
        ``out``'s tokens are known (see Scheduler.schedule_ahead); the handle is None when the
        runner has nothing to prepare for it."""
        nxt = self.scheduler.schedule_ahead(out, self.cfg.model.max_model_len)
        if nxt is None:
            return None
        self.runner.apply_copies(nxt.copies)
        return nxt, self.runner.prepare_decode([(p.seq.seq_id, p.start) for p in nxt.portions])

    @classmethod
    def from_config(cls, cfg: EngineConfig) -> "LLMEngine":
        return cls(cfg)

    def _resolve_eos(self) -> frozenset:
        """llm_engine.py:24-32: the tokenizer's eos id, else the model config's (int or list)."""
        eos = getattr(self.tokenizer, "eos_token_id", None)
        if eos is None:
            return frozenset(self.runner.spec.eos_token_ids)
        return frozenset({eos}) if isinstance(eos, int) else frozenset(eos)

    # ------------------------------------------------------------------ requests
    def add_request(self, request_id: str, prompt: Optional[str] = None,
                    sampling_params: Optional[SamplingParams] = None,
                    prompt_token_ids: Optional[list[int]] = None) -> None:
        """Queue one request; exactly one of ``prompt`` and ``prompt_token_ids`` (llm_engine.py:67-97)."""
        if (prompt is None) == (prompt_token_ids is None):
            raise ValueError("provide exactly one of prompt or prompt_token_ids")
        if request_id in self._seqs:
            raise ValueError(f"request id {request_id!r} is already active")
        if prompt_token_ids is None:
            if self.tokenizer is None:
                raise ValueError("a text prompt needs a tokenizer; pass prompt_token_ids instead")
            prompt_token_ids = self.tokenizer.encode(prompt)
        # a long prompt is checked as an array, not token by token
        ids = np.asarray(prompt_token_ids)
        if ids.ndim != 1:
            raise ValueError("prompt_token_ids must be a flat sequence of token ids")
        if ids.size == 0:
            raise ValueError("prompt must contain at least one token")
        ids = ids.astype(np.int64)
        vocab = self.runner.spec.vocab_size
        outside = (ids < 0) | (ids >= vocab)
        if outside.any():
            raise ValueError(f"token ids {ids[outside][:5].tolist()} lie outside the vocabulary [0, {vocab})")
        prompt_token_ids = ids.tolist()
        if len(prompt_token_ids) >= self.cfg.model.max_model_len:
            raise ValueError(
                f"prompt of {len(prompt_token_ids)} tokens leaves no room to generate "
                f"within max_model_len {self.cfg.model.max_model_len}"
            )
        params = sampling_params if sampling_params is not None else SamplingParams()
        if params.stop and self.tokenizer is None:
            raise ValueError("stop strings need a tokenizer; use stop_token_ids instead")
        seq = Sequence(request_id, prompt_token_ids, params, arrival_time=float(next(self._arrivals)))
        self._seqs[request_id] = seq
        self._text[request_id] = _RequestText()
        self.scheduler.add_seq(seq)

    def abort_request(self, request_id: str) -> None:
        self.scheduler.abort(request_id)
        self._forget(request_id)

    def has_unfinished_requests(self) -> bool:
        return self.scheduler.has_unfinished()

    def _forget(self, request_id: str) -> None:
        self._seqs.pop(request_id, None)
        self._text.pop(request_id, None)

    # ------------------------------------------------------------------ one iteration
    def step(self) -> list[RequestOutput]:
        """Schedule, run one batch, sample, finish; an output per request that got a token
        (llm_engine.py:99-125)."""
        started, self._started = self._started, None
        if started is not None and all(p.seq.is_finished() for p in started[0].portions):
            started = None  # queued for requests that have all stopped since: nothing of it is wanted
        if started is None:
            started = self._start_step()
            if started is None:
                return []
        out, drawn_on_device, fetch = started
        # The GPU is busy with this step: decide the next one now if it is plain decoding, and
        # put it on the GPU's queue at once, fed by this step's sampling kernels on the device,
        # so that the GPU goes from one step to the next without waiting for the host. A request
        # that stops with the token of this step is then run once too often: that costs nothing
        # but the work, its extra token is dropped and its pages are reused only by later steps.
        if self.cfg.scheduler.lookahead:
            self._ahead = self._look_ahead(out)
            if self._ahead is not None and self._ahead[1] is not None and drawn_on_device is not None:
                ahead, self._ahead = self._ahead, None
                self._started = self._start_step(ahead, device_tokens=drawn_on_device)
        tokens = self._fetched(fetch)
        drawn = iter(tokens)
        sampled: list[Sequence] = []
        may_stop = False
        for p in out.portions:
            seq = p.seq
            if seq.is_finished():  # stopped or aborted while this step was queued: its token is dropped
                if p.samples:
                    next(drawn)
                continue
            seq.num_computed_tokens = p.start + p.num_tokens
            prompt_done = p.start < len(seq.prompt_token_ids) <= seq.num_computed_tokens
            if prompt_done and self.prefix_cache.enabled:
                # the trie takes a hold only on blocks it adopts, so inserting while the
                # request still holds its pages is safe (llm_engine.py:115-119)
                n_full = len(seq.prompt_token_ids) // self.cfg.cache.block_size
                self.prefix_cache.insert(seq.prompt_token_ids, self.manager.handles(seq.seq_id, n_full))
            if p.samples:
                token = next(drawn)
                seq.append_token(token)
                sampled.append(seq)
                params = seq.sampling_params
                may_stop = may_stop or bool(params.stop) or token in params.stop_token_ids or (
                    not params.ignore_eos and token in self._eos_ids)
        # A step decided ahead that could not be queued above (no captured graph for it yet) can
        # still start before this step's outputs are made, unless a request may stop right now.
        ahead = self._ahead
        if (self._started is None and ahead is not None and not may_stop
                and ahead[0].version == self.scheduler.version):
            self._ahead = None
            self._started = self._start_step(ahead)
        outputs = [self._process(seq) for seq in sampled]
        self.scheduler.free_finished()
        for output in outputs:
            if output.finished:
                self._forget(output.request_id)
        return outputs

    def _fetching(self, drawn_on_device):
        """Begin to copy sampled tokens to the host; ``_fetched`` waits for them. The copy is
        queued before whatever the GPU is given next, so waiting for it waits for nothing else."""
        if drawn_on_device is None:
            return None
        buf = self._token_bufs[self._token_buf_at]
        self._token_buf_at ^= 1
        view = buf[: drawn_on_device.numel()]
        view.copy_(drawn_on_device, non_blocking=True)
        event = torch.cuda.Event()
        event.record()
        return view, event

    @staticmethod
    def _fetched(fetch) -> list[int]:
        if fetch is None:
            return []
        view, event = fetch
        event.synchronize()
        return view.tolist()

    def _start_step(self, ahead=None, device_tokens=None):
        """Choose a step (the one decided ahead of time if it still holds, else the scheduler's),
        put its kernels and the sampling kernels on the GPU's queue and return (schedule, sampled
        tokens as a device tensor or None, the copy of those tokens to the host under way); None
        if nothing can run. ``device_tokens``: the tokens the step before it sampled, still on
        the device and not yet appended to their requests (a step decided ahead only)."""
        if ahead is None:
            ahead, self._ahead = self._ahead, None
        if ahead is not None and ahead[0].version == self.scheduler.version:
            # decided (and mostly laid out) while the last step ran; nothing has changed since
            out, handle = ahead
            self.scheduler.commit_ahead(out)
            self.lookahead_steps += 1
        else:
            if device_tokens is not None:
                raise RuntimeError("tokens that are still on the device can only feed a step decided ahead")
            handle = None
            out = self.scheduler.schedule()
            if not out.portions:
                if out.preempted or not self.scheduler.has_unfinished():
                    return None
                # nothing runs and the head does not fit: give it everything the prefix cache
                # holds idle, once, before calling the request unschedulable (llm_engine.py:102-113)
                if self.prefix_cache.evict(self.manager.num_blocks) > 0:
                    out = self.scheduler.schedule()
                if not out.portions:
                    raise RuntimeError("waiting request cannot be admitted even with an empty prefix cache")
            self.runner.apply_copies(out.copies)
        if handle is not None:
            tokens = device_tokens if device_tokens is not None else [p.seq.output_token_ids[-1] for p in out.portions]
            logits = self.runner.step_prepared(handle, tokens)
        else:
            entries = [
                StepEntry(
                    p.seq.seq_id,
                    p.start,
                    p.seq.tokens_in(p.start, p.start + p.num_tokens),
                    [p.num_tokens - 1] if p.samples else [],
                )
                for p in out.portions
            ]
            logits = self.runner.step(entries)
        sampling = [p.seq for p in out.portions if p.samples]
        pending = 1 if device_tokens is not None else 0
        drawn = self.sampler.launch(logits, sampling, pending=pending) if sampling else None
        return out, drawn, self._fetching(drawn)

    def generate(self, prompts, sampling_params: Optional[SamplingParams] = None) -> list[RequestOutput]:
        """Run prompts (strings or lists of token ids) to completion; final outputs in prompt order
        (llm_engine.py:135-159)."""
        finals: dict[str, Optional[RequestOutput]] = {}
        for prompt in prompts:
            request_id = f"generate-{next(self._generate_ids)}"
            key = "prompt" if isinstance(prompt, str) else "prompt_token_ids"
            self.add_request(request_id, sampling_params=sampling_params, **{key: prompt})
            finals[request_id] = None
        unfinished = len(finals)
        while unfinished:
            outputs = self.step()
            for output in outputs:
                if output.finished and finals.get(output.request_id, output) is None:
                    finals[output.request_id] = output
                    unfinished -= 1
            if unfinished and not outputs and not self.scheduler.has_unfinished():
                lost = sorted(rid for rid, out in finals.items() if out is None)
                raise RuntimeError(f"the engine has nothing left to run, yet these requests never finished: {lost}")
        return list(finals.values())

    def stats(self) -> dict:
        """Counters of the scheduler and the prefix cache under the reference's names
        (llm_engine.py:161-177), and two of this engine's own."""
        report = dict(vars(self.scheduler.stats))
        cache = self.prefix_cache.stats
        for name in ("queries", "hit_tokens", "prompt_tokens", "hit_rate"):
            report[f"prefix_cache_{name}"] = getattr(cache, name)
        report["num_free_blocks"] = self.manager.min_free_blocks()
        report["lookahead_steps"] = self.lookahead_steps
        return report

    # ------------------------------------------------------------------ text and finishing
    def _decode(self, ids: list[int]) -> str:
        return self.tokenizer.decode(ids, skip_special_tokens=True)

    def _ends_with_a_stop_token(self, seq: Sequence) -> bool:
        params, token = seq.sampling_params, seq.output_token_ids[-1]
        return token in params.stop_token_ids or (token in self._eos_ids and not params.ignore_eos)

    def _is_out_of_room(self, seq: Sequence) -> bool:
        return (len(seq.output_token_ids) >= seq.sampling_params.max_tokens
                or len(seq) >= self.cfg.model.max_model_len)

    def _process(self, seq: Sequence) -> RequestOutput:
        """What the request's newest token means for it (llm_engine.py:200-242). The rules, in
        order: a stop token (end of sequence unless ``ignore_eos``, or one of ``stop_token_ids``)
        ends it, stays in the ids and adds no text; otherwise the token's text is added and a
        stop string in it ends the request with the text cut there; otherwise ``max_tokens`` or
        the model length end it with reason "length"."""
        text = self._text[seq.seq_id]
        added = ""
        if self._ends_with_a_stop_token(seq):
            seq.status = SequenceStatus.FINISHED_STOPPED
        else:
            stopped = False
            if self.tokenizer is not None:
                added, stopped = text.accept(text.grow(self._decode, seq.output_token_ids), seq.sampling_params.stop)
            if stopped:
                seq.status = SequenceStatus.FINISHED_STOPPED
            elif self._is_out_of_room(seq):
                seq.status = SequenceStatus.FINISHED_LENGTH
        reasons = {SequenceStatus.FINISHED_STOPPED: "stop", SequenceStatus.FINISHED_LENGTH: "length"}
        return RequestOutput(
            request_id=seq.seq_id,
            prompt_token_ids=seq.prompt_token_ids,  # shared, not copied: a prompt never changes
            token_ids=list(seq.output_token_ids),
            text=text.shown,
            finished=seq.is_finished(),
            finish_reason=reasons.get(seq.status),
            num_cached_tokens=seq.num_cached_tokens,
            num_prompt_tokens=len(seq.prompt_token_ids),
            num_generated_tokens=len(seq.output_token_ids),
            delta_text=added,
        )
