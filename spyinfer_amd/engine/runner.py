"""The step function: runs a batch of (request, its next tokens) from the cache
and returns logits at the wanted places.

It stands where the reference has ``ModelRunner::execute_model``
(src/engine/model_runner.cpp:49-157), but samples nothing and changes no
request: it runs only the tokens it is given, as one batch, prompt portions
beside single decoded tokens, cut anywhere.
"""
from __future__ import annotations

import gc
from typing import List, Optional, Sequence

import torch

from ..cache.manager import CacheManager
from ..cache.storage import CacheStorage
from ..config.registry import load_model_config
from ..models.base import DecoderModel
from ..weights.loader import load_weights
from .batch import StepBatch, StepEntry

DTYPES = {"bfloat16": torch.bfloat16, "float32": torch.float32, "bf16": torch.bfloat16, "fp32": torch.float32}


def resolve_dtype(name) -> torch.dtype:
    if isinstance(name, torch.dtype):
        if name not in (torch.bfloat16, torch.float32):
            raise ValueError("dtype must be bfloat16 or float32")
        return name
    if name not in DTYPES:
        raise ValueError("dtype must be 'bfloat16' or 'float32', got %r" % (name,))
    return DTYPES[name]


def bind_weights(model: DecoderModel, weights, device, weight_copies: str = "both") -> None:
    """``model.bind`` with the engine's choice of the forms in which matrices are kept (EngineConfig.weight_copies)."""
    from ..kernels import ops
    before = ops.ROW_MAJOR_WEIGHTS
    ops.ROW_MAJOR_WEIGHTS = weight_copies != "tiled"
    try:
        model.bind(weights, device)
    finally:
        ops.ROW_MAJOR_WEIGHTS = before


def load_model(folder: str, dtype, device, weight_copies: str = "both") -> DecoderModel:
    """config.json -> architecture -> model of parts, weights bound by name."""
    arch, cfg = load_model_config(folder)
    model = arch.build(cfg)
    weights = load_weights(folder, model.weight_specs(), resolve_dtype(dtype), device)
    bind_weights(model, weights, device, weight_copies)
    return model


class PreparedStep:
    """The host half of a step: its batch, planned and packed for the transfer."""
    __slots__ = ("batch", "graphable")

    def __init__(self, batch: StepBatch, graphable: bool):
        self.batch, self.graphable = batch, graphable


class ModelRunner:
    #: most step shapes that are captured as graphs
    MAX_GRAPHS = 256

    def __init__(self, model: DecoderModel, dtype, device, page_size: int, num_pages: int, max_num_seqs: int,
                 max_num_batched_tokens: int = 16384, enforce_eager: bool = True, max_model_len: Optional[int] = None):
        """``enforce_eager=False``: steps that hold single tokens only (decoding) are captured in
        HIP graphs, one per number of entries and wanted rows, and replayed; their block tables
        then have the fixed width that ``max_model_len`` needs."""
        self.model = model
        self.act_dtype = resolve_dtype(dtype)
        self.device = torch.device(device)
        self.max_num_batched_tokens = max_num_batched_tokens
        self.manager = CacheManager(model.cache_specs(), page_size, num_pages, max_num_seqs, max_num_batched_tokens)
        self.storage = CacheStorage(self.manager, self.act_dtype, self.device)
        self.steps_run = 0
        self.use_graphs = not enforce_eager
        limit = max_model_len or model.max_positions or num_pages * page_size
        self.fixed_max_blocks = min(-(-limit // page_size), max(1, num_pages))
        #: captured steps by shape; at most ``max_graphs``, further shapes run kernel by kernel.  A captured step is
        #: kept as long as the runner: none is destroyed between steps, while others may be in flight.  All captures
        #: allocate from one memory pool and write their logits into one tensor, so what they hold together is the
        #: activations of the largest step, that tensor and each graph's own copy of the step's metadata
        #: (``graph_memory_bound``): steps run one after the other on one stream, and a step's logits are read
        #: (sampled, copied) before the next step is queued.
        self._graphs = {}
        self.max_graphs = self.MAX_GRAPHS
        self.max_num_seqs = max_num_seqs
        self._graph_pool = None
        self._graph_logits = None
        self._seen = {}
        self._pinned = None
        self._copied = None
        self._packed = None        # the batch whose arrays the pinned buffer holds
        self.graph_replays = 0

    @staticmethod
    def bytes_per_page(model: DecoderModel, page_size: int, dtype) -> int:
        """Device bytes that one more page in every page group costs."""
        return CacheStorage.bytes_per_page(model.cache_specs(), page_size, resolve_dtype(dtype))

    # ---- what captured steps cost ------------------------------------------------
    @staticmethod
    def graph_logits_bytes(max_num_seqs: int, vocab_size: int) -> int:
        """The one float32 tensor [max_num_seqs, vocab] that every captured step writes its logits into."""
        return 4 * max_num_seqs * vocab_size

    @staticmethod
    def graph_metadata_bytes(entries: int, page_groups: int, fixed_max_blocks: int, plan_ints: int = 0) -> int:
        """Upper bound of a captured step's own metadata buffer: per entry a row of ``fixed_max_blocks`` page numbers
        in every page group and 64 further integers (token, position, lengths, slots; each array padded to 16 B), and
        what the model's parts plan for a step of that size (``DecoderModel.plan_ints``)."""
        return 4 * (entries * (page_groups * fixed_max_blocks + 64) + 256 + plan_ints)

    def graph_memory_bound(self, max_graphs: Optional[int] = None) -> int:
        """Most device bytes that captured steps hold beside the activations of the largest of them (which any step,
        captured or not, needs while it runs): the shared logits tensor and ``max_graphs`` metadata buffers."""
        n = self.max_graphs if max_graphs is None else max_graphs
        return self.graph_logits_bytes(self.max_num_seqs, self.model.vocab_size) \
            + n * self.graph_metadata_bytes(self.max_num_seqs, len(self.manager.page_groups), self.fixed_max_blocks,
                                            self.model.plan_ints(self.max_num_seqs))

    def prepare(self, entries: Sequence[StepEntry]) -> "PreparedStep":
        """The host work of a step that does not need the device: the batch's arrays, the checks, the parts' plans."""
        entries = list(entries)
        graphable = self.use_graphs and all(len(e.tokens) == 1 for e in entries) \
            and all(len(t) <= self.fixed_max_blocks for e in entries for t in e.cache.tables)
        batch = StepBatch(entries, self.manager, self.act_dtype, self.device, self.model.vocab_size,
                          self.fixed_max_blocks if graphable else 0)
        if batch.T > self.max_num_batched_tokens:
            raise ValueError("the step holds %d tokens, max_num_batched_tokens is %d" % (batch.T, self.max_num_batched_tokens))
        if self.model.max_positions and batch.max_kv_len > self.model.max_positions:
            raise ValueError("a request would reach %d tokens, the model's positions end at %d"
                             % (batch.max_kv_len, self.model.max_positions))
        self.model.plan(batch)
        # the parts have the last word: a part that reads the step from the host cannot be replayed from a recording
        graphable = graphable and self.model.capturable(batch)
        self._pack(batch)
        if graphable:
            batch.graph_key()
        return PreparedStep(batch, graphable)

    def step(self, entries: Sequence[StepEntry], token_source: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Run the entries' tokens as one batch.  Pages for them must have been reserved
        (``manager.reserve``).  Returns float32 logits [wanted rows, vocab] in the order of the
        entries and of their ``want`` (valid until the next step); afterwards the tokens count
        as cached.  ``token_source``: int32 [T] on the device; the step's token ids are taken from there (on the
        stream, after what produced them) instead of from the entries, whose tokens are placeholders then."""
        entries = list(entries)
        if not entries:
            return torch.empty((0, self.model.vocab_size), dtype=torch.float32, device=self.device)
        prepared = self.prepare(entries)
        batch, graphable = prepared.batch, prepared.graphable
        if token_source is not None and (token_source.dtype != torch.int32 or tuple(token_source.shape) != (batch.T,)):
            raise ValueError("token_source must be int32 [%d]" % batch.T)
        self._reset_fresh_state(batch)
        if graphable:
            logits = self._step_graph(batch, token_source)
        else:
            self._upload(batch, None)
            if token_source is not None:
                batch.token_ids.copy_(token_source)
            logits = self.model.forward(batch, self.storage)
        for e in entries:
            self.manager.commit(e.cache, len(e.tokens))
        self.steps_run += 1
        return logits

    # ---- metadata to the device ----------------------------------------------
    def _pack(self, batch: StepBatch) -> None:
        """The batch's arrays into the pinned host buffer (one buffer: the batch packed last owns it)."""
        layout, total = batch.layout()
        if self._pinned is None or self._pinned.numel() < total:
            self._pinned = torch.empty(max(total, 1 << 16), dtype=torch.int32, pin_memory=True)
            self._copied = None
        if self._copied is not None:
            self._copied.synchronize()          # the last transfer has read the pinned buffer
            self._copied = None
        batch.pack_into(self._pinned)
        batch.packed_layout, batch.packed_total = layout, total
        self._packed = batch

    def _upload(self, batch: StepBatch, dev_buf: Optional[torch.Tensor], bind: bool = True) -> None:
        """Copy the packed arrays to the device with one transfer.  ``bind=False``: the device views are not needed (a
        graph that has them is replayed)."""
        if self._packed is not batch:
            self._pack(batch)
        layout, total = batch.packed_layout, batch.packed_total
        if dev_buf is None:
            dev_buf = torch.empty(total, dtype=torch.int32, device=self.device)
        dev_buf[:total].copy_(self._pinned[:total], non_blocking=True)
        self._copied = torch.cuda.Event()
        self._copied.record()
        self._packed = None                      # the buffer is in flight until the event
        if bind:
            batch.bind_device(dev_buf, layout)

    # ---- graphs -----------------------------------------------------------------
    def _step_graph(self, batch: StepBatch, token_source: Optional[torch.Tensor] = None) -> torch.Tensor:
        key = batch.graph_key()
        held = self._graphs.get(key)
        if held is not None:
            graph, dev_buf, logits = held
            self._upload(batch, dev_buf, bind=False)
            if token_source is not None:
                off, n = batch.packed_layout["token_ids"]
                dev_buf[off:off + n].copy_(token_source)
            graph.replay()
            self.graph_replays += 1
            return logits
        if self._seen.get(key, 0) < 1 or len(self._graphs) >= self.max_graphs:
            # first step of this shape: run it kernel by kernel (this also warms the library up); so do shapes
            # beyond the number of graphs that are kept
            self._seen[key] = 1
            self._upload(batch, None)
            if token_source is not None:
                batch.token_ids.copy_(token_source)
            return self.model.forward(batch, self.storage)
        _layout, total = batch.layout()
        dev_buf = torch.empty(total, dtype=torch.int32, device=self.device)
        self._upload(batch, dev_buf)
        if token_source is not None:
            batch.token_ids.copy_(token_source)
        if self._graph_pool is None:
            self._graph_pool = torch.cuda.graph_pool_handle()
            self._graph_logits = torch.empty((self.max_num_seqs, self.model.vocab_size), dtype=torch.float32, device=self.device)
        torch.cuda.synchronize(self.device)
        graph = torch.cuda.CUDAGraph()
        out = self._graph_logits[:batch.R] if batch.R <= self.max_num_seqs else None
        # Python's cycle collector must not run inside the capture: what it frees there (dead engines, their graphs and
        # memory pools, pinned buffers) frees device memory and queries events, which HIP forbids while a stream
        # captures, and the error, raised inside a destructor, ends the process.  So the collector rests until the
        # capture is over (dead cycles wait for its next turn; collecting them here, before every capture, cost a serving
        # run with a hundred shapes more than the captures themselves).
        collecting = gc.isenabled()
        gc.disable()
        try:
            with torch.cuda.graph(graph, pool=self._graph_pool):
                logits = self.model.forward(batch, self.storage, out)
        finally:
            if collecting:
                gc.enable()
        self._graphs[key] = (graph, dev_buf, logits)
        graph.replay()                          # capture launches nothing: this replay is the step
        self.graph_replays += 1
        return logits

    def _reset_fresh_state(self, batch: StepBatch) -> None:
        """State slots of requests that run their first tokens start from zero."""
        if not self.manager.state_groups:
            return
        fresh = [e.cache.slot for e in batch.entries if e.cache.fresh]
        if not fresh:
            return
        idx = torch.tensor(fresh, dtype=torch.long, device=self.device)
        for g in self.manager.state_groups:
            for cid in g.cache_ids:
                g.spec.reset(self.storage.layer(cid), idx)
