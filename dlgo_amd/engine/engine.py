"""The step function: a batch of sequences, each bringing its next tokens (a whole
prompt, a piece of one, or a single token), run as one flat batch of rows from
the cache; logits come back for the rows that were asked for.

computerex/dlgo has two functions for one sequence, Forward(token, pos)
(models/llm/forward.go:123) and ForwardBatch(tokens, startPos)
(models/llm/forward_batch.go:78), the latter returning the last position's
logits only (:221-235).  Both write the new keys and values first and then attend
over cache rows [0, startPos+p] (:143-207), which is why a continuation is the
same computation as a prompt; the one function here relies on the same order.

There is no padding: rows of all sequences lie one after another, each with its
own position and sequence index.  A step with more rows than the workspace holds
is cut along the rows into pieces, exact by the same argument.  A step of single
tokens is captured once per batch size as a HIP graph and replayed.
"""
from __future__ import annotations

import gc
from dataclasses import dataclass, field
from typing import Callable, Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch

from .. import models as _models  # noqa: F401  (registers the architectures)
from ..cache import PAGE, Cache, CacheError, OutOfPages
from ..config import ModelConfig, build_model, load_config
from ..kernels import build as kernel_build
from ..weights import load_state, load_weights, random_tensors
from .context import StepContext, Workspace

_RUN_DTYPES = {"bfloat16": torch.bfloat16, "bf16": torch.bfloat16, "float32": torch.float32, "fp32": torch.float32,
               "f32": torch.float32}


class EngineError(RuntimeError):
    pass


def run_dtype(name) -> torch.dtype:
    if isinstance(name, torch.dtype):
        if name not in (torch.bfloat16, torch.float32):
            raise EngineError(f"the engine runs in bfloat16 or float32, not {name}")
        return name
    try:
        return _RUN_DTYPES[str(name).lower()]
    except KeyError:
        raise EngineError(f"unknown dtype {name!r}: bfloat16 or float32") from None


def recordings_bytes(vocab: int, max_batch: int = 64, graph_max_batch: int = 128, prompt_graph_bytes: int = 1 << 30,
                     use_graphs: bool = True, **_other_engine_options) -> int:
    """Device memory that an engine with these options may come to hold for its recorded steps, beyond weights, cache
    and workspace: the fixed logits of the recorded steps of single tokens, and the logits that the recordings of
    prompt steps keep (bounded by prompt_graph_bytes).  Whoever sizes a cache from the free memory takes this off first."""
    fixed = min(graph_max_batch, max(max_batch, 1)) * vocab * 4 if use_graphs else 0
    return fixed + (prompt_graph_bytes if use_graphs else 0)


def _require_gpu() -> None:
    if not torch.cuda.is_available():
        raise EngineError("no HIP device: dlgo_amd runs on an AMD GPU only and has no CPU path")


@dataclass
class Entry:
    """One sequence's part of a step: its slot, its next tokens, and the places among
    these tokens whose logits are wanted."""
    slot: int
    tokens: Sequence[int]
    want: Sequence[int] = ()


@dataclass
class _Graph:
    graph: "torch.cuda.CUDAGraph"
    batch: int
    ctx: StepContext


@dataclass
class _PromptGraph:
    graph: "torch.cuda.CUDAGraph"
    meta: torch.Tensor           # the step's int32 arrays, at the addresses the recorded kernels read
    logits: torch.Tensor         # where the recorded step leaves its logits
    ctx: StepContext


class Engine:
    def __init__(self, model, dtype="bfloat16", device="cuda:0", max_tokens: int = 8192, max_ctx: Optional[int] = None,
                 max_slots: Optional[int] = None, max_step_tokens: int = 8192, logits_rows: int = 1024,
                 use_graphs: bool = True, graph_max_batch: int = 128, prompt_graph_max_tokens: int = 4096,
                 prompt_graph_limit: int = 32, prompt_graph_bytes: int = 1 << 30):
        """`model` holds its weights already (see from_folder / from_random).  use_graphs: steps of single tokens are
        recorded per batch size, and steps of fresh prompts of up to prompt_graph_max_tokens rows per shape (the
        prompt_graph_limit most recently used shapes are kept, as long as the logits they keep stay within
        prompt_graph_bytes), the second time a size or shape is seen."""
        _require_gpu()
        self.model = model
        self.dtype = run_dtype(dtype)
        self.device = torch.device(device)
        torch.cuda.set_device(self.device)
        limit = model.config.context_length()
        pages_tokens = ((max_tokens + PAGE - 1) // PAGE) * PAGE
        self.max_ctx = min(x for x in (max_ctx, limit, pages_tokens) if x)
        self.max_step_tokens = max(1, min(max_step_tokens, pages_tokens))
        self.logits_rows = max(1, min(logits_rows, self.max_step_tokens))
        for name, part in model.named_parts():
            try:
                part.check(self.dtype)
            except ValueError as e:
                raise EngineError(f"{name}: {e}") from None
        kernel_build.ensure_built(model.kernel_variants(self.dtype))
        self.cache = Cache(model.unit_needs, max_tokens, self.max_ctx, self.dtype, self.device, max_slots,
                           self.max_step_tokens)
        self.workspace = Workspace(self.device, self.max_step_tokens)
        model.prepare(self.max_ctx, self.device)
        self.vocab = model.vocab
        # a step is recorded only if every part says its launches depend on nothing but device arrays (Part.graph_safe)
        unsafe = [name for name, part in model.named_parts() if not getattr(part, "graph_safe", True)]
        self.use_graphs = use_graphs and not unsafe
        self.eager_because = unsafe
        self.graph_max_batch = min(graph_max_batch, self.max_step_tokens)
        self._graphs: Dict[int, _Graph] = {}
        # recorded steps of fresh prompts, by shape (rows per sequence, wanted places); the least recently used one goes
        self.prompt_graph_max_tokens = prompt_graph_max_tokens
        self.prompt_graph_limit = max(1, prompt_graph_limit)
        self.prompt_graph_bytes = max(0, prompt_graph_bytes)
        self._prompt_graphs: Dict[tuple, _PromptGraph] = {}
        self._prompt_seen: Dict[tuple, int] = {}
        self._graph_seen: Dict[int, int] = {}
        self._static: Optional[Dict[str, torch.Tensor]] = None
        self._static_logits: Optional[torch.Tensor] = None
        self._meta_dev = torch.empty(0, dtype=torch.int32, device=self.device)
        self._rows_dev = torch.empty(0, dtype=torch.int32, device=self.device)
        # steps of single tokens: the sequences' page-table rows by their place in the step, per storage group, at fixed
        # addresses; (slots, version of the group's table) of what each holds
        self._seq_pages: Dict[int, torch.Tensor] = {}
        self._seq_pages_of: Dict[int, tuple] = {}
        self._staging: List[Tuple[torch.Tensor, Optional[torch.cuda.Event]]] = []
        self._staging_next = 0
        self._logits_piece: Optional[torch.Tensor] = None
        self.steps_run = 0

    # -- construction ------------------------------------------------------------
    @classmethod
    def from_folder(cls, folder: str, dtype="bfloat16", device="cuda:0", **kw) -> "Engine":
        _require_gpu()
        config = load_config(folder)
        model = build_model(config)
        load_weights(model, folder, device, run_dtype(dtype))
        return cls(model, dtype, device, **kw)

    @classmethod
    def from_random(cls, config: ModelConfig, seed: int, dtype="bfloat16", device="cuda:0", std: Optional[float] = None,
                    norm_jitter: float = 0.0, **kw) -> "Engine":
        """Random weights drawn for the seed (on the host, as a model folder written for the seed would hold them) and
        never written."""
        _require_gpu()
        model = build_model(config)
        rd = run_dtype(dtype)
        tensors = random_tensors(config, seed, rd, std, norm_jitter, device=device)
        load_state(model, tensors, device, rd, where="random weights")
        del tensors
        return cls(model, dtype, device, **kw)

    # -- slots -------------------------------------------------------------------
    def open(self, n: int = 1) -> List[int]:
        """Slots for n new sequences (all or none)."""
        if n > self.cache.n_free_slots:
            raise EngineError(f"{n} sequences asked, {self.cache.n_free_slots} slots free")
        return [self.cache.alloc_slot() for _ in range(n)]

    def fork(self, slot: int, length: Optional[int] = None) -> int:
        """A new sequence that starts as a copy of `slot` (its first `length` tokens; all by default) and goes its own
        way from there: the next step may give the two different tokens."""
        try:
            new = self.cache.copy_slot(slot, length)
        except (CacheError, OutOfPages) as e:
            raise EngineError(f"fork: {e}") from None
        self.cache.sync_tables()
        return new

    def close(self, slots: Sequence[int]) -> None:
        for s in slots:
            self.cache.free_slot(s)

    def length(self, slot: int) -> int:
        return self.cache.length(slot)

    def free_slots(self) -> int:
        return self.cache.n_free_slots

    def free_pages(self) -> Tuple[int, ...]:
        """Pages (of 64 tokens) that new sequences can still take, for each storage group of the cache (a model
        without keys and values has none)."""
        return self.cache.free_pages()

    def page_demand(self, n_tokens: int) -> Tuple[int, ...]:
        """For each storage group: the most pages a sequence that grows to n_tokens holds at any time."""
        return self.cache.page_demand(n_tokens)

    # -- uploads -----------------------------------------------------------------
    def _stage(self, n_ints: int) -> torch.Tensor:
        """A pinned host buffer that no copy in flight still reads."""
        if not self._staging:
            self._staging = [(torch.empty(max(4096, n_ints), dtype=torch.int32, pin_memory=True), None) for _ in range(4)]
        i = self._staging_next
        self._staging_next = (i + 1) % len(self._staging)
        buf, ev = self._staging[i]
        if ev is not None:
            ev.synchronize()
        if buf.numel() < n_ints:
            buf = torch.empty(n_ints * 2, dtype=torch.int32, pin_memory=True)
        self._staging[i] = (buf, None)
        return buf

    def _upload(self, fields: Dict[str, np.ndarray], dest: Optional[torch.Tensor] = None) -> Dict[str, torch.Tensor]:
        """One host-to-device copy for all the int32 arrays of a step."""
        offs, total = {}, 0
        for k, v in fields.items():
            offs[k] = total
            total += (len(v) + 3) // 4 * 4
        host = self._stage(total)
        hv = host.numpy()
        for k, v in fields.items():
            hv[offs[k]:offs[k] + len(v)] = v
        if dest is None:
            if self._meta_dev.numel() < total:
                self._meta_dev = torch.empty(total * 2, dtype=torch.int32, device=self.device)
            dest = self._meta_dev
        dest[:total].copy_(host[:total], non_blocking=True)
        ev = torch.cuda.Event()
        ev.record()
        idx = (self._staging_next - 1) % len(self._staging)
        self._staging[idx] = (self._staging[idx][0], ev)
        return {k: dest[offs[k]:offs[k] + len(v)] for k, v in fields.items()}

    def take_rows(self, x: torch.Tensor, rows: Sequence[int]) -> torch.Tensor:
        """x[rows] for rows given on the host (logits of the sequences that go on, ids of those that are fed): the row
        numbers go up with the step's arrays, the rows are picked by the library's own kernel; nothing waits."""
        from ..kernels import ops
        idx = np.asarray(rows, dtype=np.int64)
        if idx.size and (idx.min() < 0 or idx.max() >= x.shape[0]):
            raise EngineError(f"take_rows: rows {rows} of a tensor with {x.shape[0]}")
        out = torch.empty((len(idx),) + tuple(x.shape[1:]), dtype=x.dtype, device=x.device)
        if len(idx):
            stage = self._stage(len(idx))
            stage.numpy()[:len(idx)] = idx
            if self._rows_dev.numel() < len(idx):
                self._rows_dev = torch.empty(max(256, 2 * len(idx)), dtype=torch.int32, device=self.device)
            self._rows_dev[:len(idx)].copy_(stage[:len(idx)], non_blocking=True)
            ev = torch.cuda.Event()
            ev.record()
            i = (self._staging_next - 1) % len(self._staging)
            self._staging[i] = (self._staging[i][0], ev)
            ops.copy_rows(x, out, src_rows=self._rows_dev[:len(idx)])
        return out

    def _sync_seq_pages(self, slot_arr: np.ndarray) -> Dict[int, torch.Tensor]:
        """The page-table rows of these slots, in this order, on the device (one table per storage group of the cache):
        what the attention of a step of single tokens reads instead of going through the slots.  Rows go up only when
        the slots or a table changed since the last step (a new page every 64 tokens a sequence)."""
        b = len(slot_arr)
        for gi, g in enumerate(self.cache.groups):
            dev = self._seq_pages.get(gi)
            if dev is None:
                dev = torch.full((max(self.graph_max_batch, 1), g.table_host.shape[1]), -1, dtype=torch.int32, device=self.device)
                self._seq_pages[gi] = dev
            key = (g.version, slot_arr.tobytes())
            if self._seq_pages_of.get(gi) == key:
                continue
            rows = g.table_host[slot_arr]
            stage = self._stage(rows.size)
            stage.numpy()[:rows.size] = rows.reshape(-1)
            dev[:b].view(-1).copy_(stage[:rows.size], non_blocking=True)
            ev = torch.cuda.Event()
            ev.record()
            i = (self._staging_next - 1) % len(self._staging)
            self._staging[i] = (self._staging[i][0], ev)
            self._seq_pages_of[gi] = key
        return self._seq_pages

    # -- the step ----------------------------------------------------------------
    def step(self, entries: Sequence[Entry], sink: Optional[Callable[[int, torch.Tensor], None]] = None) -> Optional[torch.Tensor]:
        """Run the entries' tokens from the cache, as one batch; return float32 logits [wanted, vocab] in the
        order of the entries and of their `want` lists.  With `sink`, logits are handed over in pieces as
        sink(first_output_row, tensor) and nothing is returned (for outputs too large to keep)."""
        entries = list(entries)
        if not entries:
            raise EngineError("step: no entries")
        seen = set()
        q_lens, starts = [], []
        for e in entries:
            if e.slot in seen:
                raise EngineError(f"step: slot {e.slot} appears twice")
            seen.add(e.slot)
            try:
                start = self.cache.length(e.slot)
            except Exception as ex:
                raise EngineError(f"step: {ex}") from None
            n = len(e.tokens)
            if n < 1:
                raise EngineError(f"step: slot {e.slot} brings no tokens")
            if start + n > self.max_ctx:
                raise EngineError(f"step: slot {e.slot} would hold {start + n} tokens, the context is {self.max_ctx}")
            for w in e.want:
                if not 0 <= w < n:
                    raise EngineError(f"step: slot {e.slot} wants logits at place {w} of {n} tokens")
            q_lens.append(n)
            starts.append(start)
        tokens = np.fromiter((t for e in entries for t in e.tokens), dtype=np.int64, count=sum(q_lens))
        if tokens.min() < 0 or tokens.max() >= self.vocab:
            bad = int(tokens[(tokens < 0) | (tokens >= self.vocab)][0])
            raise EngineError(f"step: token id {bad} is outside the vocabulary of {self.vocab}")
        why = self.cache.can_reserve([(e.slot, s + n) for e, s, n in zip(entries, starts, q_lens)])
        if why:
            raise EngineError(f"step: {why}")
        self.steps_run += 1

        if (sink is None
                and all(n == 1 for n in q_lens) and all(list(e.want) == [0] for e in entries)):
            self.steps_run -= 1
            # decode() hands out a view of a buffer that the next step overwrites; a step's result is the caller's to keep
            return self.decode([e.slot for e in entries], tokens, checked=True).clone()

        # wanted rows: (output row, flat row), in output order
        cu = np.concatenate([[0], np.cumsum(q_lens)])
        wanted = [(int(cu[i]) + w) for i, e in enumerate(entries) for w in e.want]
        n_out = len(wanted)
        wanted_arr = np.asarray(wanted, dtype=np.int64)
        total = int(cu[-1])
        seq_of = np.repeat(np.arange(len(entries)), q_lens)
        pos_all = np.concatenate([np.arange(s, s + n) for s, n in zip(starts, q_lens)])

        # Fresh prompts of a shape seen before: the launches depend on the rows per sequence and the wanted places only,
        # so the step is recorded the second time the shape comes and replayed from then on.
        shape = None
        # (a recording keeps its logits: not where those would be more than 64 MB)
        if (self.use_graphs and sink is None and n_out and total <= min(self.max_step_tokens, self.prompt_graph_max_tokens)
                and n_out * self.vocab * 4 <= min(64 << 20, self.prompt_graph_bytes) and not any(starts)):
            shape = (tuple(q_lens), tuple(wanted))
        out = None
        if sink is None and (shape is None or shape not in self._prompt_graphs):
            out = torch.empty((n_out, self.vocab), dtype=torch.float32, device=self.device)

        for c0 in range(0, total, self.max_step_tokens):
            c1 = min(total, c0 + self.max_step_tokens)
            seqs = np.unique(seq_of[c0:c1])                     # sequences with rows in this piece, ascending
            local_seq = np.searchsorted(seqs, seq_of[c0:c1])
            piece_q = np.bincount(local_seq, minlength=len(seqs))
            first_row = np.concatenate([[0], np.cumsum(piece_q)[:-1]])
            piece_start = pos_all[c0:c1][first_row]
            slots = np.array([entries[int(s)].slot for s in seqs], dtype=np.int64)
            self.cache.reserve([(int(sl), int(st + q)) for sl, st, q in zip(slots, piece_start, piece_q)])
            self.cache.sync_tables()
            sel = np.nonzero((wanted_arr >= c0) & (wanted_arr < c1))[0]      # output rows served by this piece
            fields = {
                "token_ids": tokens[c0:c1].astype(np.int32),
                "positions": pos_all[c0:c1].astype(np.int32),
                "tok_seq": local_seq.astype(np.int32),
                "slots": slots.astype(np.int32),
                "start_pos": piece_start.astype(np.int32),
                "cu_q": np.concatenate([[0], np.cumsum(piece_q)]).astype(np.int32),
                "rows": (wanted_arr[sel] - c0).astype(np.int32),
            }
            host = {"q_lens": piece_q, "start_pos": piece_start, "slots": slots}
            if shape is not None:
                out = self._prompt_step(shape, fields, host, len(seqs), c1 - c0, sel, out)
            else:
                arrays = self._upload(fields)
                self._run_piece(StepContext(self, len(seqs), c1 - c0, arrays, host), arrays, sel, out, sink)
            for sl, q in zip(slots, piece_q):
                self.cache.advance(int(sl), int(q))
        return out

    def _run_piece(self, ctx: StepContext, arrays: Dict[str, torch.Tensor], sel: np.ndarray, out: Optional[torch.Tensor],
                   sink: Optional[Callable[[int, torch.Tensor], None]]) -> None:
        """The model on the rows of one piece of a step, and the logits of the wanted rows that lie in it (output rows
        `sel`), in runs of consecutive output rows of at most logits_rows each."""
        x = self.model.hidden(ctx, ctx.token_ids)
        i = 0
        while i < len(sel):
            j = i + 1
            while j < len(sel) and sel[j] == sel[j - 1] + 1 and j - i < self.logits_rows:
                j += 1
            o0 = int(sel[i])
            if out is not None:
                self.model.logits(ctx, x, arrays["rows"][i:j], out[o0:o0 + (j - i)])
            else:
                if self._logits_piece is None:
                    self._logits_piece = torch.empty((self.logits_rows, self.vocab), dtype=torch.float32, device=self.device)
                piece = self._logits_piece[:j - i]
                self.model.logits(ctx, x, arrays["rows"][i:j], piece)
                sink(o0, piece)
            i = j

    def _prompt_step(self, shape, fields: Dict[str, np.ndarray], host: Dict[str, np.ndarray], n_seq: int, n_rows: int,
                     sel: np.ndarray, out: Optional[torch.Tensor]) -> torch.Tensor:
        """A whole step of fresh prompts whose shape may be recorded: replayed if it is, recorded the second time it is
        seen, run as it is the first time.  Returns the logits (the caller's own tensor)."""
        g = self._prompt_graphs.get(shape)
        if g is not None:
            self._prompt_graphs[shape] = self._prompt_graphs.pop(shape)       # most recently used last
            self._upload(fields, dest=g.meta)
            g.graph.replay()
            return g.logits.clone()
        seen = self._prompt_seen.get(shape, 0) + 1
        self._prompt_seen[shape] = seen
        if len(self._prompt_seen) > 4096:
            self._prompt_seen.clear()
        if seen < 2:
            arrays = self._upload(fields)
            self._run_piece(StepContext(self, n_seq, n_rows, arrays, host), arrays, sel, out, None)
            return out
        total = sum((len(v) + 3) // 4 * 4 for v in fields.values())
        meta = torch.zeros(total, dtype=torch.int32, device=self.device)
        logits = torch.empty((len(sel), self.vocab), dtype=torch.float32, device=self.device)
        arrays = self._upload(fields, dest=meta)
        ctx = StepContext(self, n_seq, n_rows, arrays, host)
        graph = torch.cuda.CUDAGraph()
        torch.cuda.synchronize()
        gc.collect()
        was_enabled = gc.isenabled()
        gc.disable()            # as in _capture: nothing may be collected while the stream records
        try:
            with torch.cuda.graph(graph):
                self._run_piece(ctx, arrays, sel, logits, None)
        finally:
            if was_enabled:
                gc.enable()
        self._prompt_graphs[shape] = _PromptGraph(graph, meta, logits, ctx)
        # the least recently used recordings go when there are too many or their logits take too much
        held = lambda: sum(p.logits.numel() * 4 for p in self._prompt_graphs.values())
        while len(self._prompt_graphs) > 1 and (len(self._prompt_graphs) > self.prompt_graph_limit or held() > self.prompt_graph_bytes):
            self._prompt_graphs.pop(next(iter(self._prompt_graphs)))
        graph.replay()
        return logits.clone()

    # -- single tokens, captured ---------------------------------------------------
    def _static_arrays(self) -> Dict[str, torch.Tensor]:
        if self._static is None:
            b = self.graph_max_batch
            meta = torch.zeros(8 * b + 64, dtype=torch.int32, device=self.device)
            self._static = {"meta": meta}
            self._static_logits = torch.empty((b, self.vocab), dtype=torch.float32, device=self.device)
        return self._static

    def _decode_fields(self, tokens: np.ndarray, starts: Sequence[int], slots: Sequence[int]) -> Dict[str, np.ndarray]:
        b = len(slots)
        return {
            "token_ids": tokens.astype(np.int32),
            "positions": np.asarray(starts, dtype=np.int32),
            "slots": np.asarray(slots, dtype=np.int32),
            "start_pos": np.asarray(starts, dtype=np.int32),
            "tok_seq": np.arange(b, dtype=np.int32),
            "cu_q": np.arange(b + 1, dtype=np.int32),
        }

    def decode(self, slots: Sequence[int], tokens, checked: bool = False, replay: bool = True) -> torch.Tensor:
        """One token for each of `slots`, logits [len(slots), vocab] for each (a view that the next decode or step
        overwrites).  `tokens` are ids on the host, or an int32 tensor on the device in the order of `slots`
        (the sampler's output: the ids need not come to the host before the next step starts).  replay=False: the
        step's launches are made one by one, the same ones a recording of this batch size holds, and nothing is
        recorded (for timing them)."""
        b = len(slots)
        slot_arr = np.asarray(slots, dtype=np.int64)
        on_device = isinstance(tokens, torch.Tensor)
        if not checked:
            # the whole call, before anything runs: distinct live slots, token ids, the context, and pages for every sequence
            if b < 1:
                raise EngineError("decode: no sequences")
            if len(set(slots)) != b or slot_arr.min() < 0 or slot_arr.max() >= self.cache.max_slots \
                    or not self.cache._live[slot_arr].all():
                raise EngineError("decode: slots must be distinct and in use")
            if on_device:
                if tokens.dtype != torch.int32 or tokens.dim() != 1 or tokens.shape[0] != b or tokens.device != self.device:
                    raise EngineError("decode: device tokens must be one int32 id per slot on the engine's device")
            else:
                tok = np.asarray(tokens, dtype=np.int64)
                if tok.shape != (b,) or tok.min() < 0 or tok.max() >= self.vocab:
                    raise EngineError(f"decode: one token id inside the vocabulary of {self.vocab} per slot")
        starts = self.cache.lengths[slot_arr]
        needs_pages = bool((starts % PAGE == 0).any()) or self.cache.has_windows
        if not checked:
            if (starts + 1 > self.max_ctx).any():
                raise EngineError(f"decode: a sequence would exceed the context of {self.max_ctx}")
            if needs_pages:
                why = self.cache.can_reserve([(int(s), int(st) + 1) for s, st in zip(slot_arr, starts)])
                if why:
                    raise EngineError(f"decode: {why}")
        if b > self.graph_max_batch:
            # more sequences than the fixed arrays of a recorded step hold: in runs of that many (the call as a whole is
            # checked by now), into a buffer of this call
            out = torch.empty((b, self.vocab), dtype=torch.float32, device=self.device)
            for c0 in range(0, b, self.graph_max_batch):
                c1 = min(b, c0 + self.graph_max_batch)
                out[c0:c1].copy_(self.decode(slots[c0:c1], tokens[c0:c1], checked=True, replay=replay))
            return out
        if needs_pages:
            self.cache.reserve([(int(s), int(st) + 1) for s, st in zip(slot_arr, starts)])
            self.cache.sync_tables()
        seq_pages = self._sync_seq_pages(slot_arr)
        st = self._static_arrays()
        tok_host = np.zeros(b, dtype=np.int32) if on_device else np.asarray(tokens, dtype=np.int32)
        fields = self._decode_fields(tok_host, starts, slot_arr)
        arrays = self._upload(fields, dest=st["meta"])
        if on_device:
            arrays["token_ids"].copy_(tokens)
        logits = self._static_logits[:b]
        g = self._graphs.get(b) if self.use_graphs and replay else None
        if g is not None:
            g.graph.replay()
        else:
            host = {"q_lens": np.ones(b, dtype=np.int64), "start_pos": starts.astype(np.int64), "slots": slot_arr}
            ctx = StepContext(self, b, b, arrays, host)
            ctx.is_decode = True
            ctx.seq_pages = seq_pages
            if self.use_graphs:
                ctx.max_pages_used = self.cache.max_pages_per_seq     # the recorded launch must cover any later length
            x = self.model.hidden(ctx, ctx.token_ids, all_rows_wanted=True)
            self.model.logits(ctx, x, None, logits)
            # the second time a batch size is seen it is worth capturing
            self._graph_seen[b] = self._graph_seen.get(b, 0) + (1 if replay else 0)
            if self.use_graphs and replay and self._graph_seen[b] >= 2:
                self._capture(b, ctx, logits)
        self.cache.advance_many(slot_arr, 1)
        self.steps_run += 1
        return logits

    def _capture(self, b: int, ctx: StepContext, logits: torch.Tensor) -> None:
        """Record the step for this batch size.  Recording runs nothing; the arrays the recorded kernels
        read (token ids, positions, slots, page tables) live at fixed addresses and are refreshed before
        each replay."""
        graph = torch.cuda.CUDAGraph()
        torch.cuda.synchronize()
        # No garbage collection while recording: a collected tensor or event would make calls into the
        # runtime that a recording stream forbids, and the error is raised inside a destructor.
        gc.collect()
        was_enabled = gc.isenabled()
        gc.disable()
        try:
            with torch.cuda.graph(graph):
                x = self.model.hidden(ctx, ctx.token_ids, all_rows_wanted=True)
                self.model.logits(ctx, x, None, logits)
        finally:
            if was_enabled:
                gc.enable()
        self._graphs[b] = _Graph(graph, b, ctx)
