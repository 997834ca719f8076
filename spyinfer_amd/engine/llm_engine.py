"""The programmatic entry point, in the manner of the reference's ``LLMEngine``
(src/engine/llm_engine.hpp:18-58): add_request, append_to_request, step, is_request_finished,
remove_request, get_output_tokens, has_unfinished_requests.  Requests are token ids (the
reference tokenises text itself; tokenisation is outside this engine).  Options are the
reference's ``Config`` fields (src/config.hpp:17-30), given as keyword arguments as the
reference takes them in its parameter map (src/engine/llm_engine.cpp:11-16).
"""
from __future__ import annotations

from typing import Dict, List, NamedTuple, Optional, Sequence as Seq

import torch

from ..config.engine_config import EngineConfig
from ..sampling.sampler import Sampler, SamplingParams
from .batch import StepEntry
from ..cache.manager import CacheManager
from .runner import ModelRunner, load_model, resolve_dtype
from .scheduler import Scheduler
from .sequence import Sequence, SequenceStatus


class StepOutput(NamedTuple):
    request_id: int
    token: int
    finished: bool


class _Flight(NamedTuple):
    scheduled: list            # what the step runs (Scheduled)
    rows: list                 # (request, its cache at launch) of every sampled row, in the order of ``picked``
    picked: Optional[torch.Tensor]   # sampled token ids, on the device
    host: Optional[torch.Tensor]     # the same, on their way to the host (the copy is queued right behind the sampling,
    copied: object                   # ahead of any later step; this event tells when it is done)

    def tokens(self) -> List[int]:
        if self.picked is None:
            return []
        if self.copied is not None:
            self.copied.synchronize()
        return [int(x) for x in self.host.tolist()]


def pages_for_memory(free_bytes: int, config: EngineConfig, model) -> int:
    """Pages of the cache pool when ``free_bytes`` of device memory are free (num_kvcache_blocks not given).  From the
    free memory go first the memory that captured decode steps will hold over the run
    (``ModelRunner.graph_memory_bound``; nothing with enforce_eager); of the rest the share ``gpu_memory_utilization``
    less a tenth (the activations of one full step, the library's workspace) is the cache's.  The slots of per-request
    state are allocated whatever the pool's size, ``max_num_seqs`` of them in every layer cache that has any: they come
    off first, and if they alone do not fit, that is an error here and not an allocation failure later.  Groups of
    layers with a window get no more pages than their requests can hold (``CacheManager.pages_of_group``); what they
    leave goes to the other groups.  Never more pages than max_num_seqs requests of max_model_len tokens need."""
    page = config.kvcache_block_size
    dtype = resolve_dtype(config.dtype)
    specs = [s for s in model.cache_specs() if s is not None]
    blocks = -(-config.max_model_len // page)
    graphs = 0
    if not config.enforce_eager:
        groups = len({s for s in specs if s.paged})
        graphs = ModelRunner.graph_logits_bytes(config.max_num_seqs, model.vocab_size) \
            + ModelRunner.MAX_GRAPHS * ModelRunner.graph_metadata_bytes(config.max_num_seqs, groups, blocks,
                                                                        model.plan_ints(config.max_num_seqs))
    budget = int(max(0, free_bytes - graphs) * config.gpu_memory_utilization * 0.9)
    state = config.max_num_seqs * sum(s.page_bytes(page, dtype) for s in specs if not s.paged)
    if state > budget:
        raise ValueError("the per-request state of max_num_seqs = %d requests takes %d bytes of device memory; %d are at hand "
                         "for the cache: lower max_num_seqs" % (config.max_num_seqs, state, budget))
    budget -= state
    per_kind = {}
    for s in specs:
        if s.paged:
            per_kind[s] = per_kind.get(s, 0) + s.page_bytes(page, dtype)
    if not per_kind:
        return 1                                   # no layer keeps anything in pages
    cap = blocks * config.max_num_seqs
    pages = 0
    while per_kind:
        pages = min(cap, budget // sum(per_kind.values()))
        full = [k for k in per_kind if CacheManager.pages_of_group(k, page, max(1, pages), config.max_num_seqs,
                                                                   config.max_num_batched_tokens) < pages]
        if not full:
            break
        for k in full:          # these groups take what their windows need; the others share what is left
            budget -= per_kind.pop(k) * CacheManager.pages_of_group(k, page, pages, config.max_num_seqs, config.max_num_batched_tokens)
    return max(1, pages)


class LLMEngine:
    def __init__(self, model_path: str, device="cuda:0", **params):
        known = {f for f in EngineConfig.__dataclass_fields__}
        bad = sorted(set(params) - known)
        if bad:
            raise TypeError("unknown engine option(s): %s; known: %s" % (", ".join(bad), ", ".join(sorted(known))))
        config = EngineConfig(model=model_path, **params)
        config.validate()
        self._init_with_model(load_model(model_path, config.dtype, torch.device(device), config.weight_copies), device, **params)
        self.config.model = model_path

    def _init_with_model(self, model, device, **params) -> None:
        """Set the engine up around a model whose weights are already bound (measurements make
        their weights on the device instead of reading a folder)."""
        self.config = EngineConfig(**params)
        self.config.validate()
        self.device = torch.device(device)
        self.model = model
        mc = self.model.config
        # as the reference: a request never outgrows the model's positions (src/config.hpp:12)
        limit = self.model.max_positions or mc.position_limit
        if limit:
            self.config.max_model_len = min(self.config.max_model_len, limit)
        num_pages = self.config.num_kvcache_blocks
        if num_pages is None:
            num_pages = self._pages_from_free_memory()
        self.runner = ModelRunner(self.model, self.config.dtype, self.device, self.config.kvcache_block_size, num_pages,
                                  self.config.max_num_seqs, self.config.max_num_batched_tokens,
                                  enforce_eager=self.config.enforce_eager, max_model_len=self.config.max_model_len)
        self.scheduler = Scheduler(self.runner.manager, self.config.max_num_batched_tokens, self.config.max_num_seqs,
                                   self.config.max_model_len, self.config.prefill_chunk)
        self.sampler = Sampler(self.device)
        self.eos_token_id = -1 if mc.end_token_id is None else mc.end_token_id
        self._sequences: Dict[int, Sequence] = {}
        self._next_id = 0
        self.stats = dict(steps=0, prefill_tokens=0, decode_tokens=0)
        self._flight = None        # a step that runs on the device and whose tokens have not been read yet
        #: False: every step waits for its tokens before the next one is built (as the reference does)
        self.run_ahead = True

    def _pages_from_free_memory(self) -> int:
        free, _total = torch.cuda.mem_get_info(self.device)
        return pages_for_memory(free, self.config, self.model)

    # ---- requests --------------------------------------------------------
    def add_request(self, prompt_tokens: Seq[int], params: Optional[SamplingParams] = None) -> int:
        params = params or SamplingParams()
        params.validate()
        rid = self._next_id
        seq = Sequence(rid, [int(t) for t in prompt_tokens], params)
        for t in seq.tokens:
            if not (0 <= t < self.model.vocab_size):
                raise ValueError("token id %d is outside the vocabulary of %d" % (t, self.model.vocab_size))
        self.scheduler.add_sequence(seq)
        self._next_id += 1
        self._sequences[rid] = seq
        return rid

    def append_to_request(self, request_id: int, tokens: Seq[int], params: Optional[SamplingParams] = None) -> None:
        """A further turn of a finished request (src/engine/llm_engine.cpp:40-73).  As in the reference only the new
        tokens are computed if the request still holds its cache (``keep_finished_cache``); if its pages went back
        when it finished, or were taken back since, the history is computed again.  The tokens that come out are the
        same.  A turn that is refused (ValueError) leaves the request as it was."""
        seq = self._sequences[request_id]
        if seq.status is not SequenceStatus.FINISHED:
            raise ValueError("request %d is still running" % request_id)
        new = [int(t) for t in tokens]
        for t in new:
            if not (0 <= t < self.model.vocab_size):
                raise ValueError("token id %d is outside the vocabulary of %d" % (t, self.model.vocab_size))
        if params is not None:
            params.validate()
        turn = params if params is not None else seq.params
        self.scheduler.check_admissible(len(seq.tokens) + len(new), turn.max_new_tokens)      # raises before anything changes
        seq.draws_before += seq.num_generated
        seq.tokens += new
        seq.num_prompt_tokens = len(seq.tokens)
        seq.params = turn
        seq.finish_reason = None
        self.scheduler.add_sequence(seq)

    def is_request_finished(self, request_id: int) -> bool:
        return self._sequences[request_id].status is SequenceStatus.FINISHED

    def has_unfinished_requests(self) -> bool:
        return self.scheduler.has_unfinished()

    def get_output_tokens(self, request_id: int) -> List[int]:
        """Prompt and generated tokens, as the reference returns them (src/engine/llm_engine.cpp:139-147)."""
        return list(self._sequences[request_id].tokens)

    def get_generated_tokens(self, request_id: int) -> List[int]:
        seq = self._sequences[request_id]
        return seq.tokens[seq.num_prompt_tokens:]

    def finish_reason(self, request_id: int) -> Optional[str]:
        return self._sequences[request_id].finish_reason

    def remove_request(self, request_id: int) -> None:
        seq = self._sequences.pop(request_id)
        if seq.status is not SequenceStatus.FINISHED or seq.cache is not None:
            self.scheduler.abort(seq)

    # ---- one step --------------------------------------------------------
    def step(self) -> List[StepOutput]:
        """One step of the engine: the tokens it sampled, request by request.

        Steps in which every running request decodes one token are run ahead: before this step's tokens are read
        from the device, the next step is already launched for the same requests, its token ids handed over on the
        device (the sampler's output is copied into the next step's input).  So the device does not wait for the
        host between two such steps.  What cannot be foreseen is a request that ends at its end-of-sequence token
        (or is removed): its row in the step in flight is then ignored, and its pages, given back at once, are safe
        because whatever reuses them runs later on the same stream.  A request that ends by count is known ahead,
        and so is a request that waits for admission: no step is run ahead then."""
        flight, self._flight = self._flight, None
        if flight is not None and not any(self._alive(seq, cache) for seq, cache in flight.rows):
            flight = None                                  # every request of the step in flight has ended meanwhile
        if flight is None:
            flight = self._launch(self.scheduler.schedule())
            if flight is None:
                return []
        ahead = self._launch_ahead(flight) if self.run_ahead else None
        tokens = flight.tokens()
        outputs = []
        for (seq, cache), tok in zip(flight.rows, tokens):
            if not self._alive(seq, cache):
                continue                                   # ended or removed while the step was in flight
            seq.tokens.append(tok)
            reason = None
            # the end-of-sequence token stays in the request's tokens (src/engine/model_runner.cpp:141-151)
            if tok == self.eos_token_id and not seq.params.ignore_eos:
                reason = "eos"
            elif seq.params.max_new_tokens is not None and seq.num_generated >= seq.params.max_new_tokens:
                reason = "max_new_tokens"
            elif len(seq) >= self.config.max_model_len:
                reason = "max_model_len"
            if reason:
                self.scheduler.finish(seq, reason, keep=self.config.keep_finished_cache)
            outputs.append(StepOutput(seq.id, tok, reason is not None))
        self._flight = ahead
        return outputs

    @staticmethod
    def _alive(seq: Sequence, cache) -> bool:
        return seq.status is SequenceStatus.RUNNING and seq.cache is cache and cache.live

    def _launch(self, scheduled, token_source=None, ahead: int = 0) -> Optional["_Flight"]:
        """Run a scheduled step on the device and start its sampling; nothing waits for the device.  ``ahead`` = 1:
        the requests' newest tokens are not on the host yet (they come from ``token_source`` on the device)."""
        if not scheduled:
            return None
        entries = []
        for sc in scheduled:
            seq = sc.seq
            lo = seq.num_computed
            toks = [0] * sc.num_tokens if ahead else seq.tokens[lo:lo + sc.num_tokens]
            entries.append(StepEntry(seq.cache, toks, [sc.num_tokens - 1] if sc.samples else []))
        logits = self.runner.step(entries, token_source)
        sampling = [sc.seq for sc in scheduled if sc.samples]
        picked = self.sampler.sample_device(
            logits, [s.params.temperature for s in sampling],
            [s.params.seed if s.params.seed is not None else self.config.seed + s.id for s in sampling],
            [s.num_draws + ahead for s in sampling])
        self.stats["steps"] += 1
        for sc in scheduled:
            self.stats["decode_tokens" if sc.num_tokens == 1 and sc.samples else "prefill_tokens"] += sc.num_tokens
        host = copied = None
        if picked is not None:
            if picked.is_cuda:
                host = torch.empty(picked.shape, dtype=picked.dtype, pin_memory=True)
                host.copy_(picked, non_blocking=True)
                copied = torch.cuda.Event()
                copied.record()
            else:
                host = picked
        return _Flight(scheduled, [(s, s.cache) for s in sampling], picked, host, copied)

    def _launch_ahead(self, flight: "_Flight") -> Optional["_Flight"]:
        """The step after ``flight``, if it can be told without ``flight``'s tokens: the same requests, one token on."""
        sch = self.scheduler
        scheduled = flight.scheduled
        if sch.waiting or len(scheduled) != len(sch.running) or flight.picked is None:
            return None
        for sc in scheduled:
            seq = sc.seq
            if sc.num_tokens != 1 or not sc.samples or not self._alive(seq, seq.cache):
                return None
            # with the token of the step in flight the request goes on only if neither limit is reached
            if seq.params.max_new_tokens is not None and seq.num_generated + 1 >= seq.params.max_new_tokens:
                return None
            if len(seq) + 1 >= self.config.max_model_len:
                return None
        manager = self.runner.manager
        for sc in scheduled:
            if not manager.can_reserve(sc.seq.cache, 1):
                return None
            manager.reserve(sc.seq.cache, 1)
        return self._launch([type(sc)(sc.seq, 1, True) for sc in scheduled], flight.picked, ahead=1)

    def generate(self, prompts: Seq[Seq[int]], params: Optional[SamplingParams] = None) -> List[List[int]]:
        """Convenience loop: all prompts at once, generated tokens of each."""
        ids = [self.add_request(p, params) for p in prompts]
        while any(not self.is_request_finished(i) for i in ids):
            self.step()
        return [self.get_generated_tokens(i) for i in ids]
