"""The engine: admits requests, runs the schedule-step-sample loop, returns outputs.

Reference: LLMEngine (/root/reference/src/core/engine.rs): admission and the clipping of
max_tokens 628-806, the loop prepare_step -> run_forward -> finish_step 1034-1151 and
1363-1629, blocking generation generate_sync 1864-2011; finishing rules in
Scheduler::postprocess (/root/reference/src/core/scheduler.rs:592-661): end-of-sequence
token unless ignore_eos, max_tokens reached, max_model_len reached.  The end-of-sequence
token is not part of the output, as in the reference.
"""
from __future__ import annotations

import os
import time
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Sequence, Tuple, Union

import torch

from ..config.engine_config import (EngineConfig, GenerationConfig, GenerationOutput, Message, SamplingParams,
                                    StreamItem)
from ..sampling import Sampler, Strategy, resolve_strategy, uniform
from ..sampling.sampler import penalty_context
from ..config.model_config import ConfigError
from ..models import family_of
from .loading import load_model, parse_dtype
from .runner import ModelRunner, StepEntry
from .scheduler import Scheduler
from .tokenizer import IncrementalText, load_tokenizer

DEFAULT_MAX_TOKENS = 16384      # /root/reference/src/core/engine.rs:650-678


def _now_ms() -> int:
    return int(time.time() * 1000)


@dataclass
class _Request:
    rid: int
    tokens: List[int]                  # prompt and generated tokens
    prompt_len: int
    max_tokens: int
    params: SamplingParams
    strategy: Strategy
    seed: int
    stream: int = 0                    # which stream of random numbers of that seed
    prompt_start: int = 0
    decode_start: int = 0
    decode_finish: int = 0
    finish_reason: str = ""
    preemptions: int = 0
    stops: List[List[int]] = field(default_factory=list)    # token sequences that end the generation
    pending: int = 0                   # tokens sampled on the GPU that the host has not read yet
    closed: bool = False               # the scheduler has let go of it already (its last token is on its way)

    @property
    def generated(self) -> List[int]:
        return self.tokens[self.prompt_len:]


@dataclass
class _Launched:
    """A step that has been launched and whose sampled tokens the host has not read yet."""
    sampled: List[_Request]            # the requests of its wanted rows, in row order
    tokens: torch.Tensor               # int32 [rows] on the device
    host: torch.Tensor                 # the same in pinned memory once `ready` has happened
    ready: torch.cuda.Event
    row_of: Dict[int, int]             # request id -> its row


def plan_pages(groups: Sequence[Tuple[int, int]], page: int, max_num_seqs: int, max_model_len: int, portion: int,
               budget_bytes: int) -> List[int]:
    """Pages for every cache group.  `groups`: per group (window, bytes a token over the group's
    layers).  A group that keeps every key can use `max_num_seqs` requests of `max_model_len`
    tokens; a group with a window holds of a request the window - 1 keys before the portion that
    runs, the portion itself and one page more (they need not start at a page's edge), as the
    scheduler admits it: a model with a small window over a long context gets a small pool for
    those layers, not the context's.  If that is more than `budget_bytes`, every group gets the
    same share of what it could use (one page at least)."""
    could, size = [], []
    for window, per_token in groups:
        tokens = max_model_len
        pages = -(-tokens // page)
        if window > 0:
            pages = min(pages, -(-min(tokens, window - 1 + portion) // page) + 1)
        could.append(max_num_seqs * pages)
        size.append(max(1, per_token * page))
    if not could:
        return [1]
    need = sum(c * b for c, b in zip(could, size))
    if need <= budget_bytes:
        return [max(1, c) for c in could]
    return [max(1, int(c * budget_bytes / need)) for c in could]


class LLMEngine:
    def __init__(self, econfig: EngineConfig, dtype="bf16", model=None):
        """`model`: a loaded `CausalLM` to run instead of the folder `econfig` names (random
        weights built in memory, for measurements); the tokenizer is then the byte tokenizer."""
        self.econfig = econfig
        if model is None:
            self.dtype = parse_dtype(dtype)
            model_dir = econfig.model_dir()
            self.model = load_model(model_dir, self.dtype, econfig.device, econfig.yarn_scaling_factor)
        else:
            model_dir = None
            self.model = model
            self.dtype = model.dtype
        spec = self.model.spec
        self.max_model_len = min(econfig.max_model_len or spec.max_positions, spec.max_positions)
        try:
            default_template = family_of(spec.architecture).chat_template
        except ConfigError:                # a model put together by hand, of no registered family
            default_template = None
        self.tokenizer = load_tokenizer(model_dir, spec.vocab_size, default_template)
        self.generation_cfg = econfig.generation_cfg or (_read_generation_config(model_dir) if model_dir else None)
        # config.json's end-of-sequence ids and generation_config.json's together
        # (Config::apply_generation_cfg, /root/reference/src/utils/config.rs:360-375), and the tokenizer's
        self.eos_token_ids = set(spec.eos_token_ids) | set(self.tokenizer.eos_token_ids())
        if self.generation_cfg is not None:
            self.eos_token_ids |= set(self.generation_cfg.eos_token_id or ())
        self.seed = econfig.seed if econfig.seed is not None else int.from_bytes(os.urandom(4), "little")
        page = econfig.page_size
        num_pages = econfig.num_pages or self._plan_pages(page)
        self.runner = ModelRunner(self.model, page, num_pages, econfig.max_num_seqs,
                                  use_graphs=not econfig.disable_cuda_graph)
        budget = econfig.max_num_batched_tokens or max(econfig.prefill_chunk_size, econfig.max_num_seqs)
        self.scheduler = Scheduler(self.runner.cache, econfig.max_num_seqs, budget,
                                   econfig.prefill_chunk_size)
        self.sampler = Sampler(self.model.device)
        self._requests: Dict[int, _Request] = {}
        self._finished: Dict[int, _Request] = {}
        self._next_id = 0
        self.steps = 0
        self.num_preemptions = 0
        # set to a list to have every step's work recorded in it for a measurement: (tokens run,
        # keys in the cache of the step's requests after it, query-key pairs of its attention)
        self.step_log: Optional[list] = None
        # Running ahead: a step is launched with the tokens that the step before it is still
        # sampling (they are handed over on the device), and only then are that earlier step's
        # tokens read and its requests' stop rules applied, while the GPU works.  A request that
        # turns out to have ended (end-of-sequence, a stop sequence) has one more token computed
        # for nothing; one that reaches its length limit is known beforehand and is not planned again.
        self.run_ahead = bool(econfig.run_ahead)
        self._launched: Optional[_Launched] = None
        rows = max(1, econfig.max_num_seqs)
        self._token_pins = [torch.empty((rows,), dtype=torch.int32, pin_memory=True) for _ in range(2)]
        self._pin_turn = 0

    # ---- memory -------------------------------------------------------------------
    def _plan_pages(self, page: int) -> List[int]:
        """Pages of every cache group from a share of the memory that is free after loading the
        weights (the reference's kv_fraction, 0.6 by default on GPUs,
        /root/reference/src/utils/kvcache_allocator.rs:336-346); see `plan_pages`."""
        free, _ = torch.cuda.mem_get_info(self.model.device)
        frac = self.econfig.kv_fraction if self.econfig.kv_fraction is not None else 0.6
        esize = torch.tensor([], dtype=self.dtype).element_size()
        groups = []
        for grp in self.model.cache_groups:
            per_token = sum(pool.bytes_per_token(esize) for layer in grp.layers for pool in self.model.kv_needs[layer].pools)
            groups.append((grp.window, per_token))
        portion = min(self.econfig.prefill_chunk_size,
                      self.econfig.max_num_batched_tokens or max(self.econfig.prefill_chunk_size, self.econfig.max_num_seqs))
        return plan_pages(groups, page, self.econfig.max_num_seqs, self.max_model_len, portion, int(free * frac))

    def get_num_cached_tokens(self) -> int:
        """Tokens held by the prefix cache (xinfer.pyi:215-222): there is none here, so none."""
        return 0

    def get_available_kv_tokens(self) -> int:
        return min(self.runner.cache.free_pages(g) for g in range(len(self.runner.cache.groups))) \
            * self.econfig.page_size

    # ---- admission --------------------------------------------------------------------
    def add_request(self, prompt: Sequence[int], params: Optional[SamplingParams] = None) -> int:
        """Admits a tokenised prompt; returns the request's id."""
        params = params or SamplingParams()
        prompt = [int(t) for t in prompt]
        if not prompt:
            raise ValueError("a prompt needs at least one token")
        if len(prompt) > self.max_model_len - 1:          # engine.rs:639-647
            raise ValueError(f"prompt of {len(prompt)} tokens exceeds max_model_len {self.max_model_len}")
        vocab = self.model.spec.vocab_size
        if min(prompt) < 0 or max(prompt) >= vocab:
            raise ValueError(f"a prompt token is outside the vocabulary of {vocab}")
        max_tokens = params.max_tokens or self.econfig.max_tokens or DEFAULT_MAX_TOKENS
        max_tokens = max(1, min(max_tokens, self.max_model_len - len(prompt)))   # engine.rs:650-678
        stops: List[List[int]] = [[int(t) for t in ids] for ids in (params.stop_token_ids or []) if len(ids)]
        for text in params.stop_sequences or []:           # engine.rs:693-721: empty ones are skipped
            if text:
                ids = self.tokenizer.encode(text)
                if ids:
                    stops.append([int(t) for t in ids])
        rid = self._next_id
        self._next_id += 1
        self.scheduler.add(rid, len(prompt), max_tokens)
        # a request with a seed of its own draws from that seed's first stream whatever its
        # id; otherwise from the engine's seed and a stream of its own
        seed, stream = (params.seed, 0) if params.seed is not None else (self.seed, rid)
        self._requests[rid] = _Request(
            rid, prompt, len(prompt), max_tokens, params,
            resolve_strategy(params, self.generation_cfg), seed, stream, prompt_start=_now_ms(), stops=stops)
        return rid

    # ---- the loop ------------------------------------------------------------------------
    def step(self) -> List[int]:
        """One iteration: plan a step, launch it with its sampling, then read the tokens of the step
        launched before it and apply the finishing rules to them (with `run_ahead` off: this step's
        own).  Returns the ids that were found finished."""
        done: List[int] = []
        plan, preempted = self.scheduler.schedule()
        for rid in preempted:
            self._requests[rid].preemptions += 1
            self.num_preemptions += 1
        if self._launched is not None and (not plan or not self.run_ahead or self._needs_host_tokens(plan)):
            # the earlier step's tokens are needed before this one can be launched (or there is nothing to launch)
            done += self._collect()
            plan = [e for e in plan if e.request in self._requests]    # (the scheduler dropped the ended ones from its plan too)
        if not plan:
            if not done and not self.scheduler.idle():
                raise RuntimeError("the scheduler planned nothing although requests are waiting")
            return done
        entries, sampled = [], []
        places, rows = [], []              # tokens of this step that the launched step is still sampling
        at = 0
        for e in plan:
            r = self._requests[e.request]
            end = e.start + e.count
            if end > len(r.tokens):        # the entry's last token is on its way
                if self._launched is None or end != len(r.tokens) + 1 or r.rid not in self._launched.row_of:
                    raise RuntimeError(f"request {r.rid}: the plan runs ahead of its known tokens")
                toks = r.tokens[e.start:] + [0]
                places.append(at + e.count - 1)
                rows.append(self._launched.row_of[r.rid])
            else:
                toks = r.tokens[e.start:end]
            entries.append(StepEntry(e.request, toks, [e.count - 1] if e.sample else []))
            if e.sample:
                sampled.append(r)
            at += e.count
        device_tokens = (self._launched.tokens, places, rows) if places else None
        logits = self.runner.step(entries, reserved=True, device_tokens=device_tokens)
        self.scheduler.commit()
        self.steps += 1
        if self.step_log is not None:
            self.step_log.append((sum(e.count for e in plan), sum(e.start + e.count for e in plan),
                                  sum(e.count * e.start + e.count * (e.count + 1) // 2 for e in plan)))
        launched = None
        if sampled:
            # (a request's generated tokens are tokens[prompt_len:]; no copies of them on this path)
            strategies = [r.strategy for r in sampled]
            recent = None
            if any(s.frequency_penalty or s.presence_penalty for s in strategies):
                recent = [penalty_context(r.tokens, r.prompt_len) for r in sampled]     # (nothing is pending then)
            tokens = self.sampler.sample_device(
                logits, strategies,
                [0.0 if r.strategy.greedy else uniform(r.seed, r.stream, len(r.tokens) + r.pending - r.prompt_len)
                 for r in sampled],
                recent=recent)         # (a greedy row draws nothing)
            n = len(sampled)
            if self._token_pins[self._pin_turn].numel() < n:
                self._token_pins[self._pin_turn] = torch.empty((n,), dtype=torch.int32, pin_memory=True)
            host = self._token_pins[self._pin_turn][:n]
            self._pin_turn ^= 1
            host.copy_(tokens, non_blocking=True)
            ready = torch.cuda.Event()
            ready.record()
            launched = _Launched(sampled, tokens, host, ready, {r.rid: i for i, r in enumerate(sampled)})
            # what the scheduler needs to plan the next step is known without the tokens: every
            # sampled request grows by one, unless this token is the last it may have
            for r in sampled:
                r.pending += 1
                known = len(r.tokens) + r.pending
                if known - r.prompt_len >= r.max_tokens or known >= self.max_model_len:
                    self.scheduler.finish(r.rid)
                    r.closed = True
                else:
                    self.scheduler.append_token(r.rid)
        if self._launched is not None:
            done += self._collect()        # the step before, while the GPU runs this one
        self._launched = launched
        if launched is not None and not self.run_ahead:
            done += self._collect()
        return done

    def _needs_host_tokens(self, plan) -> bool:
        """Whether a step cannot be launched before the launched step's tokens are read: a request
        it samples for counts its recent tokens (penalties)."""
        for e in plan:
            if e.sample:
                s = self._requests[e.request].strategy
                if s.frequency_penalty or s.presence_penalty:
                    return True
        return False

    def _collect(self) -> List[int]:
        """Reads the launched step's tokens and applies the finishing rules.  Returns the ids that finished."""
        launched, self._launched = self._launched, None
        launched.ready.synchronize()
        done: List[int] = []
        now = _now_ms()
        for r, tok in zip(launched.sampled, launched.host.tolist()):
            if self._requests.get(r.rid) is not r:
                continue                   # ended or cancelled since: the token was computed for nothing
            r.pending -= 1
            if len(r.tokens) == r.prompt_len:
                r.decode_start = now
            reason = ""
            if r.stops and _completes_a_stop(r.stops, r.generated, int(tok)):
                reason = "stop"
            elif tok in self.eos_token_ids and not r.params.ignore_eos:
                reason = "eos"
            else:
                r.tokens.append(int(tok))
                if len(r.tokens) - r.prompt_len >= r.max_tokens:
                    reason = "length"
                elif len(r.tokens) >= self.max_model_len:
                    reason = "max_model_len"
            if reason:
                r.finish_reason = reason
                r.decode_finish = now
                if not r.closed:
                    self.scheduler.finish(r.rid)
                self._finished[r.rid] = self._requests.pop(r.rid)
                done.append(r.rid)
            elif r.closed and r.pending == 0:
                raise RuntimeError(f"request {r.rid} was closed but did not finish")
        return done

    def run_until_done(self) -> None:
        while not self.scheduler.idle() or self._launched is not None:
            self.step()

    # ---- outputs ---------------------------------------------------------------------------
    def _output(self, r: _Request) -> GenerationOutput:
        gen = r.generated
        return GenerationOutput(
            seq_id=r.rid, prompt_length=r.prompt_len, prompt_start_time=r.prompt_start,
            decode_start_time=r.decode_start, decode_finish_time=r.decode_finish,
            decoded_length=len(gen), decode_output=self.tokenizer.decode(gen), token_ids=list(gen),
            finish_reason=r.finish_reason)

    def generate(self, prompts: Sequence[Union[str, Sequence[int]]],
                 params: Union[SamplingParams, Sequence[SamplingParams], None] = None) -> List[GenerationOutput]:
        """Prompts as text (tokenised with the model's tokenizer) or as token ids."""
        if params is None or isinstance(params, SamplingParams):
            params = [params or SamplingParams()] * len(prompts)
        if len(params) != len(prompts):
            raise ValueError("one SamplingParams per prompt is needed")
        rids = []
        try:
            for p, sp in zip(prompts, params):
                ids = self.tokenizer.encode(p) if isinstance(p, str) else list(p)
                rids.append(self.add_request(ids, sp))
        except Exception:
            for rid in rids:               # a later prompt was refused: the earlier ones do not stay behind
                self.cancel(rid)
            raise
        self.run_until_done()
        return [self._output(self._finished.pop(rid)) for rid in rids]

    def generate_stream(self, params: SamplingParams,
                        messages: Union[Sequence[Message], str, Sequence[int]], completion: bool = False):
        """The reference's streaming entry point (xinfer.pyi:206-216): returns (seq_id,
        prompt_length, stream).  `messages` is a chat (rendered with the chat template), or a
        prompt as text or token ids.  `completion`: the stream yields one COMPLETION item when
        the request has ended instead of an item per token."""
        if isinstance(messages, str):
            ids = self.tokenizer.encode(messages)
        elif messages and isinstance(messages[0], Message):
            _text_only(messages)
            ids = self.tokenizer.encode(self.tokenizer.apply_chat_template(list(messages)))
        else:
            ids = [int(t) for t in messages]
        rid = self.add_request(ids, params)
        return rid, len(ids), EngineStream(self, rid, len(ids), completion)

    def cancel(self, rid: int) -> None:
        """Ends a request now and gives back what it holds (reference: Scheduler::cancel,
        /root/reference/src/core/scheduler.rs:780-818)."""
        r = self._requests.pop(rid, None)
        if r is None:
            self._finished.pop(rid, None)      # finished and never collected: forgotten now
            return
        if not r.closed:                       # (else the scheduler let go of it when its last token was launched)
            self.scheduler.finish(rid)
        r.finish_reason = "cancelled"
        r.decode_finish = _now_ms()

    def generate_sync(self, params: Sequence[SamplingParams],
                      message_list: Sequence[Sequence[Message]]) -> List[GenerationOutput]:
        """The reference's blocking chat entry point (xinfer.pyi:199-205): every message list
        is rendered with the chat template and completed."""
        for m in message_list:
            _text_only(m)
        prompts = [self.tokenizer.apply_chat_template(list(m)) for m in message_list]
        return self.generate(prompts, list(params))


def _text_only(messages) -> None:
    if any(getattr(m, "num_images", 0) for m in messages):
        raise ValueError("a message brings images: this engine takes text only")


def _completes_a_stop(stops: List[List[int]], generated: Sequence[int], token: int) -> bool:
    """Whether `token` after the tokens generated so far completes a stop sequence
    (scheduler.rs:1459-1490: a one-token stop matches the token; a longer one needs its first
    tokens at the end of the output)."""
    for stop in stops:
        if stop[-1] != token:
            continue
        n = len(stop) - 1
        if n == 0 or (n <= len(generated) and list(generated[len(generated) - n:]) == stop[:-1]):
            return True
    return False


class EngineStream:
    """Tokens of one request as they are generated (the reference's EngineStream,
    xinfer.pyi:182-189).  Iterating drives the engine: every step also advances whatever other
    requests are live.  Each token comes as a TOKEN_ID item followed by a TOKEN item with the text
    it adds (empty while a character that spans several tokens is incomplete: the text is
    decoded from all tokens so far and handed on up to where it is final); text still held back
    when the request ends comes as one more TOKEN item, so that the pieces joined are the text of
    all tokens; the last item is DONE.  With `completion` nothing comes until the request has
    ended, and then one COMPLETION item with its times and all its token ids (the reference's
    item for requests that are not streamed, /root/reference/src/core/engine.rs:64-70,1486-1492).
    A stream that is dropped unread takes its request's record with it."""

    def __init__(self, engine: "LLMEngine", rid: int, prompt_length: int, completion: bool = False):
        self._engine = engine
        self._completion = bool(completion)
        self.seq_id = rid
        self.prompt_length = prompt_length
        self.finished = False
        self.cancelled = False
        self._sent = 0
        self._text = IncrementalText(engine.tokenizer)
        self._pending: List[StreamItem] = []

    def cancel(self) -> None:
        if not self.finished and not self.cancelled:
            self._engine.cancel(self.seq_id)
            self.cancelled = True

    def __del__(self):
        try:
            self.cancel()
        except Exception:
            pass

    def __iter__(self):
        return self

    def __next__(self) -> StreamItem:
        eng = self._engine
        while not self._pending:
            if self.finished or self.cancelled:
                raise StopIteration
            r = eng._requests.get(self.seq_id) or eng._finished.get(self.seq_id)
            if r is None:
                self.finished = True
                return StreamItem("ERROR", f"request {self.seq_id} is gone")
            gen = r.generated
            if self._completion:
                if self.seq_id in eng._finished:
                    eng._finished.pop(self.seq_id)
                    self.finished = True
                    return StreamItem("COMPLETION", (r.prompt_start, r.decode_start, r.decode_finish, list(gen)))
                eng.step()
                continue
            if self._sent < len(gen):
                tok = gen[self._sent]
                self._sent += 1
                self._pending = [StreamItem("TOKEN", self._text.add(gen[:self._sent]))]
                return StreamItem("TOKEN_ID", tok)
            if self.seq_id in eng._finished:
                eng._finished.pop(self.seq_id)
                self.finished = True
                done = StreamItem("DONE", (r.prompt_start, r.decode_start, r.decode_finish, len(gen)))
                rest = self._text.finish(gen)
                if rest:
                    self._pending = [done]
                    return StreamItem("TOKEN", rest)
                return done
            eng.step()
        return self._pending.pop(0)


def _read_generation_config(model_dir: str) -> Optional[GenerationConfig]:
    import json
    path = os.path.join(model_dir, "generation_config.json")
    if not os.path.isfile(path):
        return None
    with open(path, "r", encoding="utf-8") as f:
        raw = json.load(f)
    eos = raw.get("eos_token_id")
    if eos is None:
        eos = ()
    elif isinstance(eos, int):
        eos = (eos,)
    return GenerationConfig(raw.get("temperature"), raw.get("top_p"), raw.get("top_k"),
                            raw.get("frequency_penalty"), raw.get("presence_penalty"),
                            eos_token_id=tuple(int(t) for t in eos))
