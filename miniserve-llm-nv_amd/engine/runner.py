"""The step function: a batch of (request, its next tokens) in, logits at the
wanted places out.  It runs only the tokens it is given, as one batch, from the
cache that earlier steps left, inside a cache transaction
(reference for the transaction: miniserve/engine/core.py:317-434; for executing a
plan: miniserve/engine/executor.py:239-255, which runs one forward per request
where this runs one for all).
"""

from __future__ import annotations

import gc
import weakref

import numpy as np
from dataclasses import dataclass
from pathlib import Path
from typing import Sequence

import torch

from ..cache import CacheLayout, CacheManager, StepItem
from ..config import EngineConfig, load_config
from ..parts.model import TORCH_DTYPES, DecoderModel
from ..weights import WeightLoadReport, load_weights, random_model_tensors
from ..parts.base import GroupStepView, HostBatch, StepContext
from .batch import BuiltStep, StepEntry, build_step


def _require_gpu(device: torch.device) -> None:
    if device.type != "cuda" or not torch.cuda.is_available():
        raise RuntimeError("the engine runs on the GPU only (HIP kernels); no CPU path exists.")


def recorded_batch_size(batch: int) -> int:
    """The size of the recorded step that serves ``batch`` single tokens: 1, 2, 4, 8,
    then the next multiple of 4 up to 32, of 8 up to 128, of 16 beyond.  A server's
    batch shrinks and grows by ones; recording a step for every size it passes
    through would cost more than the few spare rows do."""

    if batch <= 8:
        return 1 << (batch - 1).bit_length()
    step = 4 if batch <= 32 else 8 if batch <= 128 else 16
    return -(-batch // step) * step


def recorded_context_bound(longest: int, limit: int) -> int:
    """The context bound of the recorded step that serves rows of up to ``longest``
    tokens: 256, 512, 1024, ... up to ``limit`` (the longest request the engine admits).
    Kernels inside a recording size their launches by the bound (the parts that the keys
    of a row are cut into, say), and the block tables have its width, so a short context
    is not served by a step made for the longest one; a request that grows past a bound
    moves on to the next recording."""

    bound = 256
    while bound < longest:
        bound *= 2
    return min(bound, limit)


_SPARE_ROW = object()       # marks a row of a host buffer that holds the values of a spare row


class DecodeGraph:
    """One decode step of a fixed batch size and context bound, recorded as a HIP graph.

    A step in which every request brings one token launches a few hundred small
    kernels; recorded once and replayed, the launches cost next to nothing.  The
    integer metadata of the step lives in one static device buffer that every
    replay reads; a step copies its own values there (one copy from pinned host
    memory) and replays.  Block tables have the static width of the step's context
    bound.  The graph holds no memset node: nothing in the recorded step clears memory.
    Integer tables that parts ask for (``step_tables``) are made once, from what holds
    for every replay, and lie in the same buffer.

    A step of fewer requests than ``batch`` fills the other rows with spare ones:
    token 0 at position 0 of a sequence whose only page is the pools' spare page and
    whose state slot is the spare slot.  They write and read nothing that a request
    holds, and their logits are not returned.
    """

    def __init__(self, runner: "ModelRunner", batch: int, bound: int) -> None:
        self.batch = batch
        self.bound = bound
        # no strong reference back: a runner that is dropped goes at once, with its graphs,
        # and not at some later collection of cycles
        self._runner = weakref.ref(runner)
        groups = len(runner.cache.layout.groups)
        widths = tuple(-(-bound // size) for size in runner.cache.block_sizes)     # per group: pages of a row at the bound
        # the parts' own tables, from what every replay shares: one token a row
        host_batch = HostBatch((1,) * batch, tuple(range(batch + 1)), None, batch, recorded=True)
        part_tables = {name: np.asarray(values, dtype=np.int64)
                       for name, values in runner.model.step_tables(host_batch).items()}
        sizes = [("token_ids", batch), ("positions", batch), ("seq_of_token", batch), ("query_start", batch + 1),
                 ("context_lens", batch), ("state_slots", batch), ("logit_rows", batch)]
        sizes += [(f"part:{name}", values.size) for name, values in part_tables.items()]
        for group in range(groups):
            sizes += [(f"slots{group}", batch), (f"table{group}", batch * widths[group])]
        # for a step launched behind the sampling of the step before: which of that step's rows each row continues
        sizes += [("token_rows", batch)]
        self.offsets: dict[str, tuple[int, int]] = {}
        total = 0
        for name, size in sizes:
            self.offsets[name] = (total, size)
            total += size
        # two host buffers, used in turn: the next step's numbers may be written while the
        # copy of this step's is still on its way
        self.hosts = [torch.zeros(total, dtype=torch.int32).pin_memory() for _ in range(2)]
        self.hosts_np = [host.numpy() for host in self.hosts]
        for host in self.hosts_np:
            for name, values in part_tables.items():
                start, size = self.offsets[f"part:{name}"]
                host[start : start + size] = values
        self._turn = 0
        self.meta = torch.zeros(total, dtype=torch.int32, device=runner.device)
        self.widths = widths
        view = lambda name: self.meta[self.offsets[name][0] : self.offsets[name][0] + self.offsets[name][1]]
        self.ctx = StepContext(
            num_tokens=batch,
            num_seqs=batch,
            token_ids=view("token_ids"),
            positions=view("positions"),
            seq_of_token=view("seq_of_token"),
            query_start=view("query_start"),
            context_lens=view("context_lens"),
            state_slots=view("state_slots"),
            groups=[
                GroupStepView(block_table=view(f"table{g}").view(batch, widths[g]), slot_mapping=view(f"slots{g}"))
                for g in range(groups)
            ],
            # what holds for every replay: one token a row.  Launch decisions inside the
            # graph go by the bound; per-request numbers live on the device only.
            query_lens=[1] * batch,
            query_start_host=list(range(batch + 1)),
            context_lens_host=None,
            state_slots_host=None,
            first_positions_host=None,
            decode_prefix=batch,
            recorded=True,
            context_bound=bound,
            tables={name: view(f"part:{name}") for name in part_tables},
        )
        self.rows = view("logit_rows")
        # the table object that each row of the host buffer was last filled from: a request's
        # table is the same object until it gets a page, so most steps rewrite no row
        self._row_tables: list[list[list[object]]] = [[[None] * batch for _ in range(groups)] for _ in range(2)]
        self.graph: torch.cuda.CUDAGraph | None = None
        self.logits: torch.Tensor | None = None
        self.replays = 0

    def _next_buffer(self) -> int:
        which = self._turn
        self._turn ^= 1
        return which

    def _fill(self, reservation, which: int) -> None:
        """Everything of the step but its token ids, into host buffer ``which``."""

        host, offsets, batch = self.hosts_np[which], self.offsets, self.batch

        def put(name: str, values) -> None:
            start, size = offsets[name]
            host[start : start + size] = values

        metas = reservation.sequences
        spare = batch - len(metas)
        if spare < 0:
            raise ValueError(f"{len(metas)} requests do not fit a recorded step of {batch}.")
        if any(meta.after > self.bound for meta in metas):
            raise ValueError(f"a request is longer than the {self.bound} tokens this recorded step was made for.")
        runner = self._runner()
        put("positions", [meta.before for meta in metas] + [0] * spare)
        put("seq_of_token", range(batch))
        put("query_start", range(batch + 1))
        put("context_lens", [meta.after for meta in metas] + [1] * spare)
        put("state_slots", [meta.state_slot for meta in metas] + [runner.cache.spare_state_slot] * spare)
        put("logit_rows", range(batch))
        for group in range(len(runner.cache.layout.groups)):
            pool_pages = runner.cache.num_blocks[group]
            block_size, width = runner.cache.block_sizes[group], self.widths[group]
            slots = []
            start, _ = offsets[f"table{group}"]
            row_tables = self._row_tables[which][group]
            for row, meta in enumerate(metas):
                table = meta.block_tables[group]
                slot = meta.slot_mappings[group][0]
                page = table[meta.before // block_size]
                if not 0 <= page < pool_pages or slot != page * block_size + meta.before % block_size:
                    raise RuntimeError(f"request {meta.request_id!r}: slot {slot} disagrees with its block table.")
                slots.append(slot)
                if row_tables[row] is not table:
                    # a page that was given back is never read; 0 keeps the entry inside the pool
                    host[start + row * width : start + row * width + len(table)] = [p if p >= 0 else 0 for p in table]
                    row_tables[row] = table
            spare_page = runner.cache.spare_page(group)
            for row in range(len(metas), batch):
                slots.append(spare_page * block_size)
                if row_tables[row] is not _SPARE_ROW:
                    host[start + row * width] = spare_page
                    row_tables[row] = _SPARE_ROW
            put(f"slots{group}", slots)

    def prepare(self, reservation) -> int | None:
        """Fills a host buffer for a coming step whose token ids are not known yet and
        returns its number; None when the step is not recorded yet."""

        if self.graph is None:
            return None
        which = self._next_buffer()
        self._fill(reservation, which)
        return which

    def run(self, entries: Sequence[StepEntry], reservation, prepared: int | None = None) -> torch.Tensor:
        """Logits ``[len(entries), vocab]`` of the step; the tensor is a view of the
        graph's own output buffer and holds these values until the next step of this
        recorded size.  ``prepared``: the host buffer that :meth:`prepare` filled for
        this reservation."""

        which = prepared
        if which is None:
            which = self._next_buffer()
            self._fill(reservation, which)
        start, size = self.offsets["token_ids"]
        self.hosts_np[which][start : start + size] = [entry.token_ids[0] for entry in entries] + [0] * (size - len(entries))
        self.meta.copy_(self.hosts[which], non_blocking=True)
        runner = self._runner()
        model, views = runner.model, runner._call_views
        if self.graph is None:
            # Once eagerly, so that libraries set themselves up outside the recording.  The
            # replay below runs the same step again: cache slots are written twice with the
            # same values, and per-request state is put back to what it was before the step.
            model.forward(self.ctx, views, self.rows)
            runner.cache.restore_state(reservation)
            torch.cuda.synchronize(runner.device)
            self.ctx.scratch.clear()        # what the step shares between layers is made again inside the recording
            graph = torch.cuda.CUDAGraph()
            # No collection of cycles while the stream records: it may free what earlier
            # owners left behind (pinned memory, other graphs), and a free is not allowed
            # inside a recording - the process would abort.
            collecting = gc.isenabled()
            gc.disable()
            try:
                with torch.cuda.graph(graph, pool=runner._graph_pool):
                    self.logits = model.forward(self.ctx, views, self.rows)
            finally:
                if collecting:
                    gc.enable()
            self.graph = graph
        self.graph.replay()
        self.replays += 1
        return self.logits[: len(entries)]

    def launch_chained(self, which: int, tokens: torch.Tensor, count: int, source_rows: Sequence[int] | None = None) -> None:
        """Replays the step whose numbers :meth:`prepare` wrote into host buffer ``which``
        with the token ids of its first ``count`` rows taken from ``tokens`` (int32, on
        the device: what the sampling kernel of the step before chose) instead of from the
        host, which has not read them yet: row ``i`` runs ``tokens[i]``, or
        ``tokens[source_rows[i]]`` when the step before had other rows or another order
        (a request of it has ended, say).  Rows that only fill the step up keep the ids
        they had (any id inside the vocabulary serves them)."""

        start, size = self.offsets["token_ids"]
        if start != 0 or self.graph is None:
            raise RuntimeError("a chained step needs its recording, and the token ids at the front of its numbers.")
        if source_rows is not None:
            # the map goes to the device with the step's other numbers, in the same copy
            map_start, _ = self.offsets["token_rows"]
            self.hosts_np[which][map_start : map_start + count] = source_rows
        self.meta[size:].copy_(self.hosts[which][size:], non_blocking=True)
        if source_rows is None:
            self.meta[:count].copy_(tokens[:count])
        else:
            self.meta[:count].copy_(torch.index_select(tokens, 0, self.meta[map_start : map_start + count].long()))
        self.graph.replay()
        self.replays += 1


@dataclass
class PreparedDecode:
    """A step of single tokens whose cache transaction is open and whose numbers are
    written, but for the token ids.  ``launched``: it runs already, its token ids fed on
    the device from the sampling of the step before (:meth:`ModelRunner.launch_chained`)."""

    request_ids: tuple[str, ...]
    reservation: object
    buffer: int
    launched: bool = False


@dataclass(frozen=True)
class PreparedStep:
    """Any other step whose cache transaction is open and whose tensors are made, but
    for the single tokens that were not known yet; ``admitted``: the requests that
    were admitted for it."""

    request_ids: tuple[str, ...]
    reservation: object
    built: BuiltStep
    admitted: tuple[str, ...]


class ModelRunner:
    """Owns the model, its weights and the cache; offers ``step``."""

    def __init__(
        self,
        model: DecoderModel,
        tensors: dict[str, torch.Tensor],
        engine_config: EngineConfig,
        *,
        device: torch.device | str = "cuda:0",
    ) -> None:
        self.device = torch.device(device)
        _require_gpu(self.device)
        from .. import ops

        ops.load()
        if model.dtype == torch.bfloat16:
            # the library product's binding and workspace, before the pool is sized from what is free
            ops.prepare_products(self.device)
        self.model = model
        self.spec = model.spec
        self.engine_config = engine_config.validate(max_positions=self.spec.max_positions)
        self.dtype = model.dtype
        if TORCH_DTYPES[self.engine_config.dtype] != self.dtype:
            raise ValueError("the model and the engine configuration disagree on the dtype.")
        model.load_weights(tensors)
        self.max_model_len = self.engine_config.resolved_max_model_len(self.spec.max_positions)
        self.block_size = self.engine_config.kv_block_size
        layout = CacheLayout.from_needs(model.cache_needs())
        num_blocks = self.engine_config.num_kv_blocks
        if num_blocks is None:
            num_blocks = self._blocks_from_free_memory(layout)
        if num_blocks * self.block_size >= 2**31:
            raise ValueError("the cache pool is too large for 32-bit slot numbers.")
        self.cache = CacheManager(
            layout,
            block_size=self.block_size,
            num_blocks=num_blocks,
            max_num_seqs=self.engine_config.max_num_seqs,
            max_model_len=self.max_model_len,
        )
        self.cache.allocate_storage(self.dtype, self.device)
        self._call_views = self.cache.call_views()
        self._decode_graphs: dict[tuple[int, int], DecodeGraph] = {}     # by (rows, context bound)
        self._graph_pool = None
        self.steps_run = 0
        self.tokens_run = 0
        self.graph_steps = 0
        self.prepared_steps = 0        # steps whose numbers were written while the step before ran
        self.prepared_mixed_steps = 0  # those of them that are not recorded steps
        self.chained_steps = 0         # recorded steps launched before the host had read the tokens they run
        self.voided_chained_steps = 0  # those of them that were thrown away (a request of theirs had ended)
        self.mapped_chained_steps = 0  # those of them whose tokens were taken through a map of rows

    # ---- construction -----------------------------------------------------------------
    @classmethod
    def from_folder(
        cls, model_dir: str | Path, engine_config: EngineConfig, *, device: torch.device | str = "cuda:0"
    ) -> "ModelRunner":
        """A folder with ``config.json`` and safetensors; the model class is chosen
        by ``config.json: architectures``."""

        _require_gpu(torch.device(device))
        config = load_config(model_dir)
        model = DecoderModel(config.model_spec(), engine_config.dtype)
        tensors, report = load_weights(model_dir, model.weight_specs(), dtype=model.dtype, device=device)
        runner = cls(model, tensors, engine_config, device=device)
        runner.config = config
        runner.load_report = report
        return runner

    @classmethod
    def from_random(
        cls, config, engine_config: EngineConfig, *, seed: int = 0, device: torch.device | str = "cuda:0"
    ) -> "ModelRunner":
        """Random weights from ``seed``: a small model gets the values that
        ``write_random_model`` writes for the seed, a large one is drawn on the device."""

        _require_gpu(torch.device(device))
        model = DecoderModel(config.model_spec(), engine_config.dtype)
        tensors = random_model_tensors(model.weight_specs(), seed=seed, dtype=model.dtype, device=device)
        runner = cls(model, tensors, engine_config, device=device)
        runner.config = config
        runner.load_report = WeightLoadReport(model_dir="<random>")
        return runner

    def _blocks_from_free_memory(self, layout: CacheLayout) -> int:
        """Pages that fit into 80% of the memory that is free after the weights,
        but no more than ``max_num_seqs`` full-length requests need."""

        torch.cuda.empty_cache()      # what loading left behind (the unstacked matrices) goes back to the device first
        free_bytes, _ = torch.cuda.mem_get_info(self.device)
        itemsize = torch.empty((), dtype=self.dtype).element_size()
        per_block = max(layout.bytes_per_token(itemsize) * self.block_size, 1)
        by_memory = int(free_bytes * 0.8) // per_block
        by_need = self.engine_config.max_num_seqs * -(-self.max_model_len // self.block_size)
        blocks = max(1, min(by_memory, by_need))
        return blocks

    def _recorded_step_key(self, batch: int, longest: int) -> tuple[int, int]:
        """(rows, context bound) of the recorded step that serves ``batch`` single tokens
        whose longest row has ``longest`` tokens after the step."""

        return recorded_batch_size(batch), recorded_context_bound(longest, self.max_model_len)

    def _decode_graph_step(self, entries: Sequence[StepEntry], reservation, prepared: int | None = None) -> torch.Tensor | None:
        """A step of single tokens through the recorded graph of its batch size.  The
        graph computes the logits of every row; the wanted ones are picked."""

        for entry in entries:
            if entry.token_ids[0] >= self.spec.vocab_size:
                raise ValueError(f"entry {entry.request_id!r}: a token id is outside the vocabulary.")
        batch = len(entries)
        key = self._recorded_step_key(batch, max(meta.after for meta in reservation.sequences))
        graph = self._decode_graphs.get(key)
        if graph is None:
            if self._graph_pool is None:
                self._graph_pool = torch.cuda.graph_pool_handle()
            graph = self._decode_graphs[key] = DecodeGraph(self, *key)
        logits = graph.run(entries, reservation, prepared)
        wanted = [index for index, entry in enumerate(entries) if entry.want]
        if len(wanted) == batch:
            return logits
        if not wanted:
            return None
        return logits[torch.tensor(wanted, device=self.device)]

    # ---- requests -------------------------------------------------------------------
    def admit(self, request_id: str) -> int:
        return self.cache.admit(request_id)

    def release(self, request_id: str) -> None:
        self.cache.release(request_id)

    # ---- the step ---------------------------------------------------------------------
    def prepare_decode(self, request_ids: Sequence[str]) -> "PreparedDecode | None":
        """Opens the cache transaction of a coming step in which each of these requests
        brings one token that is not known yet, and fills the recorded step's numbers
        for it, so that :meth:`step` has only the token ids left to do.  None when such a
        step is not served from a recording (then nothing is opened).  The result goes
        to :meth:`step` with entries for the same requests in the same order, or to
        :meth:`discard`."""

        if not self.engine_config.decode_graphs or not request_ids:
            return None
        items = []
        for request_id in request_ids:
            start = self.cache.committed_tokens(request_id)
            items.append(StepItem(request_id, start, start + 1))
        graph = self._decode_graphs.get(self._recorded_step_key(len(items), max(item.end for item in items)))
        if graph is None or graph.graph is None:
            return None
        reservation = self.cache.prepare_step(items)
        try:
            buffer = graph.prepare(reservation)
        except BaseException:
            self.cache.abort_step(reservation)
            raise
        return PreparedDecode(tuple(request_ids), reservation, buffer)

    def prepare_step(self, entries: Sequence[StepEntry], admit: Sequence[str] = ()) -> "PreparedStep":
        """Opens the cache transaction of a coming step and makes its tensors, without
        sending them: entries that bring one token may bring any token id here, the
        true one is taken from the entries that :meth:`step` gets.  ``admit``: requests
        of the step that are not admitted yet.  On an exception nothing is kept."""

        admitted: list[str] = []
        try:
            for request_id in admit:
                self.admit(request_id)
                admitted.append(request_id)
            reservation = self._open_step(entries)
            try:
                built = build_step(
                    entries, reservation, block_sizes=self.cache.block_sizes, pool_pages=self.cache.num_blocks,
                    vocab_size=self.spec.vocab_size, device=self.device, step_tables=self.model.step_tables,
                )
            except BaseException:
                self.cache.abort_step(reservation)
                raise
        except BaseException:
            for request_id in admitted:
                self.release(request_id)
            raise
        return PreparedStep(tuple(entry.request_id for entry in entries), reservation, built, tuple(admitted))

    @torch.inference_mode()
    def launch_chained(self, prepared: "PreparedDecode", tokens: torch.Tensor, source_rows: Sequence[int] | None = None) -> None:
        """Launches the prepared step of single tokens now, behind the step that is still
        running: row ``i`` runs ``tokens[i]`` (int32 on the device, the sampling kernel's
        output of the running step), or ``tokens[source_rows[i]]`` when the running step's
        rows are not this step's requests in this order.  The host reads those tokens
        afterwards; :meth:`step` with this ``prepared`` then launches nothing and returns
        the logits, and :meth:`discard` throws the step away (it is a transaction like any
        other: what it wrote lies above the committed lengths, its pages and state rows go
        back)."""

        if prepared.launched:
            raise RuntimeError("the step runs already.")
        rows = len(prepared.request_ids)
        if tokens.dtype != torch.int32 or tokens.ndim != 1 or not tokens.is_cuda:
            raise ValueError("a chained step takes the device's int32 tokens, one a request.")
        if source_rows is None:
            if tokens.numel() < rows:
                raise ValueError("a chained step takes the device's int32 tokens, one a request.")
        elif len(source_rows) != rows or any(not 0 <= row < tokens.numel() for row in source_rows):
            raise ValueError("a chained step's row map names one row of the tokens for each of its requests.")
        metas = prepared.reservation.sequences
        graph = self._decode_graphs[self._recorded_step_key(len(metas), max(meta.after for meta in metas))]
        graph.launch_chained(prepared.buffer, tokens, len(metas), source_rows)
        prepared.launched = True
        self.chained_steps += 1
        self.mapped_chained_steps += source_rows is not None

    def discard(self, prepared: "PreparedDecode | PreparedStep") -> None:
        """Gives back what :meth:`prepare_decode` or :meth:`prepare_step` took."""

        if getattr(prepared, "launched", False):
            self.voided_chained_steps += 1
        self.cache.abort_step(prepared.reservation)
        for request_id in getattr(prepared, "admitted", ()):
            self.release(request_id)

    def _open_step(self, entries: Sequence[StepEntry]):
        items = []
        for entry in entries:
            start = self.cache.committed_tokens(entry.request_id)
            items.append(StepItem(entry.request_id, start, start + len(entry.token_ids)))
        return self.cache.prepare_step(items)

    @torch.inference_mode()
    def step(self, entries: Sequence[StepEntry], prepared: "PreparedDecode | None" = None) -> torch.Tensor | None:
        """Run one batch.  Every request of ``entries`` must be admitted; its tokens
        continue where its committed tokens end.  Returns float32 logits
        ``[wanted, vocab]`` in the order of the entries and of their ``want``, or
        None when nothing is wanted.  On an exception the step leaves no trace in
        the cache manager.  ``prepared``: what :meth:`prepare_decode` returned for
        exactly these requests."""

        if not entries:
            raise ValueError("a step needs at least one entry.")
        if isinstance(prepared, PreparedStep):
            return self._run_prepared_step(entries, prepared)
        if prepared is not None:
            if tuple(entry.request_id for entry in entries) != prepared.request_ids or any(
                len(entry.token_ids) != 1 for entry in entries
            ):
                self.cache.abort_step(prepared.reservation)
                raise ValueError("the entries are not those the step was prepared for.")
            reservation = prepared.reservation
            self.prepared_steps += 1
        else:
            reservation = self._open_step(entries)
        if prepared is not None and prepared.launched:
            # the step runs already (launch_chained): its logits lie in its recording's output
            metas = reservation.sequences
            graph = self._decode_graphs[self._recorded_step_key(len(metas), max(meta.after for meta in metas))]
            self.cache.commit_step(reservation)
            self.steps_run += 1
            self.tokens_run += len(entries)
            self.graph_steps += 1
            wanted = [index for index, entry in enumerate(entries) if entry.want]
            if len(wanted) == len(entries):
                return graph.logits[: len(entries)]
            return graph.logits[torch.tensor(wanted, device=self.device)] if wanted else None
        if self.engine_config.decode_graphs and all(len(entry.token_ids) == 1 for entry in entries):
            try:
                logits = self._decode_graph_step(entries, reservation, None if prepared is None else prepared.buffer)
            except BaseException:
                self.cache.abort_step(reservation)
                raise
            self.cache.commit_step(reservation)
            self.steps_run += 1
            self.tokens_run += len(entries)
            self.graph_steps += 1
            return logits
        try:
            built = build_step(
                entries,
                reservation,
                block_sizes=self.cache.block_sizes,
                pool_pages=self.cache.num_blocks,
                vocab_size=self.spec.vocab_size,
                device=self.device,
                step_tables=self.model.step_tables,
            )
            built.send()
            logits = self.model.forward(built.ctx, self._call_views, built.rows)
        except BaseException:
            self.cache.abort_step(reservation)
            raise
        self.cache.commit_step(reservation)
        self.steps_run += 1
        self.tokens_run += built.ctx.num_tokens
        return logits

    def _run_prepared_step(self, entries: Sequence[StepEntry], prepared: PreparedStep) -> torch.Tensor | None:
        """The step that :meth:`prepare_step` made, with the single tokens of ``entries``."""

        built = prepared.built
        try:
            if tuple(entry.request_id for entry in entries) != prepared.request_ids or tuple(
                len(entry.token_ids) for entry in entries
            ) != built.query_lens_of_entries:
                raise ValueError("the entries are not those the step was prepared for.")
            for index, entry in enumerate(entries):
                if len(entry.token_ids) == 1:
                    built.set_single_token(index, entry.token_ids[0])
            built.send()
            logits = self.model.forward(built.ctx, self._call_views, built.rows)
        except BaseException:
            self.cache.abort_step(prepared.reservation)
            raise
        self.cache.commit_step(prepared.reservation)
        self.steps_run += 1
        self.tokens_run += built.ctx.num_tokens
        self.prepared_steps += 1
        self.prepared_mixed_steps += 1
        return logits
