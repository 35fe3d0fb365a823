"""The step function: one call runs one batch of (request, its next tokens) through
the model, from the cache, and returns the logits at the wanted places.

A batch may hold portions of prompts beside single decoded tokens, cut anywhere;
both are the same case here: a span of new tokens behind a cached prefix.  The
reference runs two separate forwards instead, whole prompts through
`prefill_batch` and single tokens through `decode_batch`
(src/mini_llm_runtime/qwen_model_runner.py:296-376, 447-508; engine.py:186-248),
and has no partial prompts.  What is kept from it: the cache transaction around the
forward (commit only after the head succeeded, abort on any exception,
qwen_model_runner.py:371-375, 495-503), result rows in the order of the batch
(engine.py:256-260) and the position bound (qwen_model_runner.py:319-320, 474-475).
"""

from __future__ import annotations

import warnings
from dataclasses import dataclass, field
from types import SimpleNamespace
from typing import Any, Optional, Sequence

import numpy as np
import torch

from ..cache.manager import CacheManager, StepLayout
from ..parts.context import MixerPlan, PlanInput, StepContext
from ..parts.model import DecoderModel



@dataclass(frozen=True)
class StepEntry:
    """A request's next tokens and the places among them whose logits are wanted."""

    request_id: str
    tokens: tuple[int, ...]
    want: tuple[int, ...] = ()

    @staticmethod
    def of(request_id: str, tokens: Sequence[int], want: Sequence[int] = ()) -> "StepEntry":
        return StepEntry(request_id, tuple(int(t) for t in tokens), tuple(int(w) for w in want))


@dataclass
class StepOutput:
    """logits: [K, vocab] float32 on the device (None when nothing was wanted), in the
    order of the entries and of each entry's `want`; `rows[i]` = (request, index).
    They are the caller's to keep, unless the step was asked for with `borrow_logits=True`
    (or launched with `launch_decode`): then they may be a view of a recorded step's output
    buffer, which the next step of the same shape overwrites.
    site_outputs: with `capture_sites=True`, [sites, K, hidden] float32: the residual stream
    after every execution site at the wanted rows."""

    logits: Optional[torch.Tensor]
    rows: tuple[tuple[str, int], ...]
    layout: StepLayout
    passed_pages: dict = field(default_factory=dict)
    site_outputs: Optional[torch.Tensor] = None


def _pack_int32(arrays: Sequence[np.ndarray]) -> tuple[np.ndarray, list[tuple[int, tuple[int, ...]]]]:
    """Concatenate int32 arrays into one buffer (each start 16-byte aligned)."""
    spans = []
    at = 0
    for a in arrays:
        spans.append((at, a.shape))
        at += (a.size + 3) // 4 * 4
    buf = np.zeros(max(at, 4), dtype=np.int32)
    for (start, shape), a in zip(spans, arrays):
        buf[start : start + a.size] = a.reshape(-1)
    return buf, spans


class ModelRunner:
    def __init__(
        self,
        model: DecoderModel,
        cache: CacheManager,
        ops: Any,
        *,
        use_graphs: bool = True,
        max_graph_batch: int = 256,
        max_decode_graphs: int = 64,
        max_step_graphs: int = 16,
        max_graph_tokens: int = 8192,
    ) -> None:
        if model.embed_weight is None:
            raise ValueError("the model's parameters are not loaded")
        self.model = model
        self.cache = cache
        self.ops = ops
        self.device = cache.device
        self.dtype = cache.dtype
        self.vocab_size = model.spec.vocab_size
        self.max_positions = model.spec.max_position_embeddings
        self.fail_next_step: Optional[BaseException] = None  # test hook: raise inside the forward
        specs = model.site_cache_specs()
        if tuple(specs) != tuple(cache.site_specs):
            raise ValueError("the cache manager was built for another model's sites")
        self._pinned = torch.cuda.is_available() and self.device.type == "cuda"
        # Steps that hold single tokens only are captured once per (padded batch, table
        # width) as a HIP graph and replayed: a decode step of a small model is hundreds of
        # short kernels, and launching them one by one from the host costs more than running them.
        # Only for models whose parts all say `replayable`; fixed-size state is no obstacle (its
        # rows come with the step's uploaded metadata, padded entries use the banks' spare rows).
        # (a recording runs the parts' host code once, so their reports to the visibility check
        # would be missing from every replay: the check runs unrecorded)
        self.use_graphs = bool(use_graphs) and self.device.type == "cuda" and not cache.check_visibility
        self.max_graph_batch = int(max_graph_batch)
        self._graphs: dict[tuple[int, int], tuple] = {}
        self._staging: dict[tuple[int, int], list] = {}
        # Any other step (prompt portions, mixed batches) is recorded when its sizes come a second
        # time, and replayed from then on, if every part of the model allows it; a bounded number
        # of such recordings is kept, the least recently used one goes first.
        self.max_step_graphs = int(max_step_graphs)
        self.max_decode_graphs = int(max_decode_graphs)
        self.max_graph_tokens = int(max_graph_tokens)
        self._step_graphs: dict[tuple, tuple] = {}
        self._step_seen: dict[tuple, int] = {}
        # One mixer per plan key makes the step's plan under that key (mixers that share a key
        # make the same plan from the same shape), found once with a probe shape.
        probe = PlanInput(np.ones(1, dtype=np.int32), np.zeros(1, dtype=np.int32), cache.block_size)
        self._planners: dict[Any, Any] = {}
        for entry in model.spec.order:
            mixer = model.layers[entry.layer].mixer
            plan = mixer.plan(ops, probe)
            if plan is not None and plan.key not in self._planners:
                self._planners[plan.key] = mixer
        self._replayable = bool(model.replayable)  # the parts are fixed from here on

    # -------------------------------------------------------------------------------------------
    def _validate(self, entries: Sequence[StepEntry]) -> np.ndarray:
        """Checks the entries and returns their token ids as one int32 array."""
        if not entries:
            raise ValueError("a step needs at least one entry")
        ids = []
        for e in entries:
            if not e.tokens:
                raise ValueError(f"request {e.request_id!r}: no tokens in this step")
            # prompts come in thousands of tokens: types and bounds are checked without a Python
            # loop over them, which runs only to name the offender
            tokens = np.asarray(e.tokens, dtype=np.int64) if set(map(type, e.tokens)) == {int} else None
            if tokens is None or tokens.min() < 0 or tokens.max() >= self.vocab_size:
                for t in e.tokens:
                    if isinstance(t, bool) or not isinstance(t, int) or not 0 <= t < self.vocab_size:
                        raise ValueError(
                            f"request {e.request_id!r}: token {t!r} is outside the vocabulary of {self.vocab_size}"
                        )
                raise ValueError(f"request {e.request_id!r}: bad tokens")
            ids.append(tokens)
            for w in e.want:
                if not 0 <= w < len(e.tokens):
                    raise ValueError(f"request {e.request_id!r}: wanted place {w} is outside its {len(e.tokens)} tokens")
            cached = self.cache.get_request(e.request_id).num_tokens
            if cached + len(e.tokens) > self.max_positions:
                raise ValueError(
                    f"request {e.request_id!r}: {cached + len(e.tokens)} tokens exceed "
                    f"max_position_embeddings={self.max_positions}"
                )
        return np.concatenate(ids).astype(np.int32)

    # ---- metadata of a step ------------------------------------------------------------------
    FIXED_ARRAYS = 9  # token ids, positions, token entries, cu_q, q_starts, context lengths, state rows (2), wanted rows

    def _plans(self, shape: PlanInput) -> list[MixerPlan]:
        """The launch plans of the model's mixers for a step of this shape, one per plan key, in
        the order of the sites.  The step function uploads their arrays and keys its recordings
        by their sizes; what is in them is the mixers' business."""
        plans = []
        for key, mixer in self._planners.items():
            plan = mixer.plan(self.ops, shape)
            if plan is None or plan.key != key:
                raise RuntimeError(f"the mixer that plans {key!r} made no plan under that key for a step's shape")
            plans.append(plan)
        return plans

    @staticmethod
    def _plan_sizes(plans: Sequence[MixerPlan]) -> tuple:
        return tuple((repr(p.key), tuple(sorted(p.sizes.items()))) for p in plans)

    def _arrays(
        self,
        layout: StepLayout,
        token_ids: np.ndarray,
        logit_rows: np.ndarray,
        plans: Sequence[MixerPlan],
        pad_entries: Optional[int] = None,
        table_width: Optional[int] = None,
    ) -> list[np.ndarray]:
        """The int32 arrays a step uploads, in a fixed order: the FIXED_ARRAYS, a slot mapping
        and a block table per page pool, then the plans' arrays.  With `pad_entries` (a batch
        of single tokens only) every array is padded to that many entries: padded entries
        have no cached tokens, write nothing (slot -1, the state banks' spare rows) and own no
        page.  With `table_width` the block tables are that wide."""
        planned = [np.ascontiguousarray(a, dtype=np.int32) for p in plans for a in p.arrays.values()]
        tables = layout.block_tables
        if table_width is not None:
            rows = pad_entries if pad_entries is not None else layout.num_entries
            wide_tables = []
            for t in tables:
                wide = np.full((rows, table_width), -1, dtype=np.int32)
                wide[: t.shape[0], : t.shape[1]] = t
                wide_tables.append(wide)
            tables = wide_tables
        if pad_entries is None:
            return [
                token_ids, layout.positions, layout.token_entry, layout.cu_q, layout.q_starts,
                layout.context_lens, layout.state_read, layout.state_write, logit_rows,
                *layout.slot_mappings, *tables, *planned,
            ]
        count, padded = layout.num_entries, pad_entries

        def pad(a: np.ndarray, fill: int) -> np.ndarray:
            out = np.full(padded, fill, dtype=np.int32)
            out[:count] = a
            return out

        spare_read, spare_write = self.cache.state_spare_rows
        return [
            pad(token_ids, 0), pad(layout.positions, 0), np.arange(padded, dtype=np.int32),
            np.arange(padded + 1, dtype=np.int32), pad(layout.q_starts, 0), pad(layout.context_lens, 0),
            pad(layout.state_read, spare_read), pad(layout.state_write, spare_write), np.arange(padded, dtype=np.int32),
            *[pad(m, -1) for m in layout.slot_mappings], *tables, *planned,
        ]

    def _context(self, dev: torch.Tensor, spans, layout: Optional[StepLayout], plans: Sequence[MixerPlan], **sizes) -> StepContext:
        groups = len(self.cache.groups)

        def view(i: int) -> torch.Tensor:
            start, shape = spans[i]
            n = int(np.prod(shape)) if shape else 1
            return dev[start : start + n].view(shape)

        ctx = StepContext(
            ops=self.ops,
            dtype=self.dtype,
            device=self.device,
            token_ids=view(0),
            positions=view(1),
            token_entry=view(2),
            cu_q=view(3),
            q_starts=view(4),
            context_lens=view(5),
            host=layout,
            **sizes,
        )
        state_read, state_write = view(6), view(7)
        ctx.memo["logit_rows"] = view(8)
        first = self.FIXED_ARRAYS
        slot_maps = [view(first + g) for g in range(groups)]
        tables = [view(first + groups + g) for g in range(groups)]
        at = first + 2 * groups
        for plan in plans:
            fields: dict[str, Any] = dict(plan.sizes)
            for name in plan.arrays:
                fields[name] = view(at)
                at += 1
            ctx.plans[plan.key] = SimpleNamespace(**fields)
        # every site's view is made by the spec of the site whose cache it uses: the step function
        # does not know what kinds of cache there are
        for site in range(self.model.num_sites):
            source = self.model.cache_site_of(site)
            view = self.cache.site_view(site, source, tables, slot_maps, state_read, state_write)
            if view is not None:
                ctx.site_views[site] = view
        return ctx

    def _stage(self, arrays: list[np.ndarray]):
        buf, spans = _pack_int32(arrays)
        host = torch.from_numpy(buf)
        if self._pinned:
            host = host.pin_memory()
        return host, spans

    def _forward_eager(
        self,
        layout: StepLayout,
        token_ids: np.ndarray,
        logit_rows: np.ndarray,
        site_outputs: Optional[list] = None,
    ) -> Optional[torch.Tensor]:
        longest = int(layout.context_lens.max())
        plans = self._plans(PlanInput(layout.q_lens, layout.q_starts, longest, layout, token_ids))
        host, spans = self._stage(self._arrays(layout, token_ids, logit_rows, plans))
        dev = host.to(self.device, non_blocking=True)
        ctx = self._context(
            dev,
            spans,
            layout,
            plans,
            num_tokens=layout.num_tokens,
            num_entries=layout.num_entries,
            max_q_len=int(layout.q_lens.max()),
            max_context_len=longest,
        )
        return self.model.forward(ctx, ctx.memo["logit_rows"] if logit_rows.size else None, site_outputs)

    # ---- steps of sizes seen before, as HIP graphs ----------------------------------------------------
    def _table_quantum(self) -> int:
        return max(1, 1024 // self.cache.block_size)  # table widths in steps of 1,024 tokens

    def _table_width(self, layout: StepLayout) -> int:
        pages = -(-int(layout.context_lens.max()) // self.cache.block_size)
        quantum = self._table_quantum()
        return -(-pages // quantum) * quantum

    def _recordable(self) -> bool:
        return self.use_graphs and self._replayable

    def _recording_ran_out_of_memory(self, error: BaseException) -> None:
        """A recording (its private activations and logits buffer) did not fit beside the weights
        and the page pool: every recording is dropped, which frees their memory, and steps run
        unrecorded from here on."""
        self.use_graphs = False
        self._graphs.clear()
        self._step_graphs.clear()
        self._staging.clear()
        self._step_seen.clear()
        if self.device.type == "cuda":
            torch.cuda.empty_cache()
        warnings.warn(
            f"recording a step as a HIP graph ran out of device memory ({error}); recordings are switched off "
            "and every step launches its kernels one by one, which is slower.  Give the page pool less memory "
            "(num_blocks, kv_memory_fraction) or lower the GraphLimits.",
            RuntimeWarning,
            stacklevel=3,
        )

    def _step_key(self, layout: StepLayout, logit_rows: np.ndarray, token_ids: Optional[np.ndarray] = None) -> Optional[tuple]:
        """(identity of a recording, the plans it was derived from): the sizes that fix every launch
        of a step; None when such steps are not recorded."""
        if not self._recordable() or layout.num_tokens > self.max_graph_tokens:
            return None
        width = self._table_width(layout)
        plans = self._plans(PlanInput(layout.q_lens, layout.q_starts, width * self.cache.block_size, layout, token_ids))
        key = ("step", layout.num_tokens, layout.num_entries, width, int(logit_rows.size), self._plan_sizes(plans))
        return key, plans

    def _forward_recorded(
        self, key: tuple, plans: Sequence[MixerPlan], layout: StepLayout, token_ids: np.ndarray, logit_rows: np.ndarray
    ) -> Optional[torch.Tensor]:
        """Replay (recording first, if need be) the graph of a step of these sizes."""
        width = key[3]
        arrays = self._arrays(layout, token_ids, logit_rows, plans, table_width=width)
        graph = self._step_graphs.pop(key, None)
        if graph is None:
            buf, spans = _pack_int32(arrays)
            static = torch.empty(buf.size, dtype=torch.int32, device=self.device)
            static.copy_(torch.from_numpy(buf))
            ctx = self._context(
                static,
                spans,
                None,  # what a recording bakes in must not come from this one step's layout
                plans,
                num_tokens=layout.num_tokens,
                num_entries=layout.num_entries,
                max_q_len=layout.num_tokens,
                max_context_len=width * self.cache.block_size,
            )
            wanted = ctx.memo["logit_rows"] if logit_rows.size else None
            # one plain run with exactly these launch sizes first: whatever is set up at a
            # kernel's first use must exist before the recording (the run writes the same cache
            # entries the replay will write again)
            self.model.forward(ctx, wanted)
            torch.cuda.synchronize(self.device)
            ctx.memo = {"logit_rows": ctx.memo["logit_rows"]}
            captured = torch.cuda.CUDAGraph()
            with torch.cuda.graph(captured):
                out = self.model.forward(ctx, wanted)
            graph = (captured, static, out, spans, buf.size)
            while len(self._step_graphs) >= self.max_step_graphs:
                oldest = next(iter(self._step_graphs))
                del self._step_graphs[oldest]
                self._staging.pop(oldest, None)
        self._step_graphs[key] = graph  # most recently used last
        captured, static, out, spans, size = graph
        slot = self._graph_staging(key, spans, size)
        for view, array in zip(slot[1], arrays):
            view[...] = array.reshape(view.shape)
        static.copy_(slot[0], non_blocking=True)
        if self._pinned:
            done = slot[2] or torch.cuda.Event()
            done.record(torch.cuda.current_stream(self.device))
            slot[2] = done
        captured.replay()
        return out

    # ---- decode steps as HIP graphs ---------------------------------------------------------------
    def _graph_key(self, layout: StepLayout) -> Optional[tuple[int, int]]:
        """(padded batch, block table width) when the step can replay a captured graph."""
        if not self._recordable() or (layout.q_lens != 1).any():
            return None
        count = layout.num_entries
        if count > self.max_graph_batch:
            return None
        padded = 1
        while padded < count:
            padded *= 2
        return padded, self._table_width(layout)

    def _graph_staging(self, key: tuple, spans, size: int):
        """Two pinned host buffers per graph (a step fills one while the other may still be
        read by the previous step's copy), each with int32 views in the order of `_arrays`."""
        staging = self._staging.get(key)
        if staging is None:
            buffers = []
            for _ in range(2):
                host = torch.zeros(size, dtype=torch.int32, pin_memory=self._pinned)
                flat = host.numpy()
                views = [flat[start : start + (int(np.prod(shape)) if shape else 1)].reshape(shape) for start, shape in spans]
                buffers.append([host, views, None])
            staging = [buffers, 0]
            self._staging[key] = staging
        buffers, turn = staging
        staging[1] = turn ^ 1
        slot = buffers[turn]
        if slot[2] is not None:
            slot[2].synchronize()  # the copy that last read this buffer
        return slot

    def _padded_plans(
        self, padded: int, width: int, layout: Optional[StepLayout] = None, token_ids: Optional[np.ndarray] = None
    ) -> list[MixerPlan]:
        """Plans of a batch of `padded` single tokens whose contexts fit `width` pages."""
        starts = np.zeros(padded, dtype=np.int32)
        if layout is not None:
            starts[: len(layout.q_starts)] = layout.q_starts
        return self._plans(
            PlanInput(np.ones(padded, dtype=np.int32), starts, width * self.cache.block_size, layout, token_ids)
        )

    def _fill_padded(self, views, layout: StepLayout, token_ids: np.ndarray, graph) -> None:
        """`_arrays(..., pad_entries, table_width)` written into the views of a staging buffer.
        The views of the constant arrays (token_entry, cu_q, logit rows) were set when the
        buffer was made."""
        count = layout.num_entries
        spare_read, spare_write = self.cache.state_spare_rows
        for view, values, fill in (
            (views[0], token_ids, 0), (views[1], layout.positions, 0), (views[4], layout.q_starts, 0),
            (views[5], layout.context_lens, 0), (views[6], layout.state_read, spare_read),
            (views[7], layout.state_write, spare_write),
        ):
            view[:count] = values
            view[count:] = fill
        groups = len(layout.slot_mappings)
        first = self.FIXED_ARRAYS
        for g in range(groups):
            view = views[first + g]
            view[:count] = layout.slot_mappings[g]
            view[count:] = -1
            table = views[first + groups + g]
            t = layout.block_tables[g]
            table[:count, : t.shape[1]] = t
            table[:count, t.shape[1] :] = -1
            table[count:] = -1
        padded, width, sizes, has_plan_arrays = graph[5]
        if has_plan_arrays:  # plans whose arrays depend on the step's data are made again
            plans = self._padded_plans(padded, width, layout, token_ids)
            if self._plan_sizes(plans) != sizes:
                raise RuntimeError("a mixer's plan for a batch of single tokens changed its sizes between steps")
            at = first + 2 * groups
            for plan in plans:
                for array in plan.arrays.values():
                    views[at][...] = np.asarray(array, dtype=np.int32).reshape(views[at].shape)
                    at += 1

    def _forward_graph(
        self, key: tuple[int, int], layout: StepLayout, token_ids: np.ndarray, logit_rows: np.ndarray
    ) -> torch.Tensor:
        padded, width = key
        graph = self._graphs.pop(key, None)
        if graph is None:
            plans = self._padded_plans(padded, width, layout, token_ids)
            arrays = self._arrays(layout, token_ids, logit_rows, plans, padded, width)
            buf, spans = _pack_int32(arrays)
            slot = self._graph_staging(key, spans, buf.size)
            for other in self._staging[key][0]:
                other[0].numpy()[:] = buf  # the constant arrays, once
            static = torch.empty(buf.size, dtype=torch.int32, device=self.device)
            static.copy_(slot[0], non_blocking=True)
            ctx = self._context(
                static,
                spans,
                None,
                plans,
                num_tokens=padded,
                num_entries=padded,
                max_q_len=1,
                max_context_len=width * self.cache.block_size,
                logits_for_all=True,
            )
            # one eager run first: everything that is set up lazily must exist before capture
            self.model.forward(ctx, ctx.memo["logit_rows"])
            torch.cuda.synchronize(self.device)
            ctx.memo = {"logit_rows": ctx.memo["logit_rows"]}
            captured = torch.cuda.CUDAGraph()
            with torch.cuda.graph(captured):
                out = self.model.forward(ctx, ctx.memo["logit_rows"])
            has_plan_arrays = any(np.asarray(a).size for p in plans for a in p.arrays.values())
            graph = (captured, static, out, spans, buf.size, (padded, width, self._plan_sizes(plans), has_plan_arrays))
            # nothing is running here (the plain run above was waited for): the graphs that
            # were used longest ago can go
            while len(self._graphs) >= self.max_decode_graphs:
                oldest = next(iter(self._graphs))
                del self._graphs[oldest]
                self._staging.pop(oldest, None)
        self._graphs[key] = graph  # most recently used last
        out = self._replay(key, graph, layout, token_ids, None)
        if logit_rows.size == layout.num_entries and (logit_rows == np.arange(layout.num_entries)).all():
            return out[: layout.num_entries]
        if logit_rows.size == 0:
            return None
        return out[torch.from_numpy(logit_rows.astype(np.int64)).to(self.device)]

    def _replay(self, key, graph, layout: StepLayout, token_ids: np.ndarray, device_tokens: Optional[torch.Tensor]):
        """Upload the step's metadata into the graph's static buffer and replay it; token ids
        come from the host array or, stream-ordered after the upload, from a device tensor."""
        captured, static, out, spans, size = graph[:5]
        slot = self._graph_staging(key, spans, size)
        self._fill_padded(slot[1], layout, token_ids, graph)
        static.copy_(slot[0], non_blocking=True)
        if self._pinned:
            done = slot[2] or torch.cuda.Event()
            done.record(torch.cuda.current_stream(self.device))
            slot[2] = done
        if device_tokens is not None:
            start = spans[0][0]
            static[start : start + layout.num_entries].copy_(device_tokens)
        captured.replay()
        return out

    # ---- a decode step launched ahead of its tokens ---------------------------------------------------
    @torch.inference_mode()
    def launch_decode(self, request_ids: Sequence[str], device_tokens: torch.Tensor) -> Optional[StepOutput]:
        """Launch one token per request whose ids are still on the device (the sampler's output
        of the step before), without waiting for them on the host.  The step's pages are taken
        but nothing counts until `commit`; `abort` gives them back (whatever the GPU then still
        writes lands in pages that later steps, ordered behind it on the stream, overwrite).
        Returns None when such a step cannot replay an already captured graph."""
        count = len(request_ids)
        if not self._recordable() or not 0 < count <= self.max_graph_batch:
            return None
        if device_tokens.shape != (count,) or device_tokens.dtype != torch.int32 or device_tokens.device != self.device:
            raise ValueError("device_tokens must be int32 [requests] on the runner's device")
        for rid in request_ids:
            if self.cache.get_request(rid).num_tokens + 1 > self.max_positions:
                return None
        layout = self.cache.begin_step([(rid, 1) for rid in request_ids])
        try:
            key = self._graph_key(layout)
            graph = self._graphs.pop(key, None) if key is not None else None
            if graph is None:
                self.cache.abort_step()
                return None
            self._graphs[key] = graph  # most recently used last
            out = self._replay(key, graph, layout, np.zeros(count, dtype=np.int32), device_tokens)
        except BaseException:
            self.cache.abort_step()
            raise
        return StepOutput(logits=out[:count], rows=tuple((rid, 0) for rid in request_ids), layout=layout)

    def commit(self, launched: StepOutput) -> StepOutput:
        """Make a step from `launch_decode` count."""
        launched.passed_pages = self.cache.commit_step()
        return launched

    def abort(self, launched: StepOutput) -> None:
        """Give back what a step from `launch_decode` took."""
        self.cache.abort_step()

    # -------------------------------------------------------------------------------------------
    @torch.inference_mode()
    def step(
        self, entries: Sequence[StepEntry], *, borrow_logits: bool = False, capture_sites: bool = False
    ) -> StepOutput:
        """Run one batch.  borrow_logits: the caller uses the logits before the next step and
        accepts a view of a recorded step's buffer (saves a copy).  capture_sites: also return
        the residual stream after every site at the wanted rows (runs unrecorded)."""
        token_ids = self._validate(entries)
        layout = self.cache.begin_step([(e.request_id, len(e.tokens)) for e in entries])
        try:
            rows: list[tuple[str, int]] = []
            flat: list[int] = []
            for r, e in enumerate(entries):
                for w in e.want:
                    rows.append((e.request_id, w))
                    flat.append(int(layout.cu_q[r]) + w)
            logit_rows = np.asarray(flat, dtype=np.int32)
            if self.fail_next_step is not None:
                error, self.fail_next_step = self.fail_next_step, None
                raise error
            captured: Optional[list] = [] if capture_sites else None
            borrowed = False
            key = None if capture_sites else self._graph_key(layout)
            if key is not None:
                try:
                    logits = self._forward_graph(key, layout, token_ids, logit_rows)
                    borrowed = True
                except torch.cuda.OutOfMemoryError as error:
                    self._recording_ran_out_of_memory(error)
                    logits = self._forward_eager(layout, token_ids, logit_rows)
            elif capture_sites:
                logits = self._forward_eager(layout, token_ids, logit_rows, captured)
            else:
                keyed = self._step_key(layout, logit_rows, token_ids)
                seen = 0
                if keyed is not None:
                    seen = self._step_seen[keyed[0]] = self._step_seen.get(keyed[0], 0) + 1
                    if len(self._step_seen) > 4096:
                        self._step_seen.clear()
                if seen >= 2:
                    try:
                        logits = self._forward_recorded(keyed[0], keyed[1], layout, token_ids, logit_rows)
                        borrowed = True
                    except torch.cuda.OutOfMemoryError as error:
                        self._recording_ran_out_of_memory(error)
                        logits = self._forward_eager(layout, token_ids, logit_rows)
                else:
                    logits = self._forward_eager(layout, token_ids, logit_rows)
            if borrowed and not borrow_logits and logits is not None:
                logits = logits.clone()
        except BaseException:
            self.cache.abort_step()
            raise
        passed = self.cache.commit_step()
        sites = torch.stack(captured) if captured else None
        return StepOutput(logits=logits, rows=tuple(rows), layout=layout, passed_pages=passed, site_outputs=sites)
