"""A decoder made of parts: embedding, layers, the order in which the layers run,
final norm and output head.

The run order is data: a list of LayerRun entries.  An entry names the layer to
run and, optionally, an earlier entry whose cache it reads instead of keeping its
own; a layer may appear more than once (each appearance then has a cache unit of
its own unless it reads another's).  For the Llama decoder the list is simply
layers 0..L-1 (computerex/dlgo, models/llm/forward.go:137-184).
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Iterator, List, Optional, Sequence, Tuple

import torch

from .base import CacheNeed, Part, TensorSpec
from .block import Block
from .embedding import Embedding, OutputHead
from .position import PositionEncoding


@dataclass(frozen=True)
class LayerRun:
    layer: int                          # index into the model's layers
    reads_cache_of: Optional[int] = None   # index into the run order of the entry whose cache is read


class DecoderModel:
    def __init__(self, config, embedding: Tuple[str, Embedding], layers: Sequence[Tuple[str, Block]],
                 final_norm: Tuple[str, Part], head: Tuple[str, OutputHead], order: Optional[Sequence[LayerRun]] = None,
                 position: Optional[Tuple[str, PositionEncoding]] = None, ignorable_tensors: Sequence[str] = ()):
        self.config = config
        self.embedding_name, self.embedding = embedding
        self.layers = list(layers)
        self.final_norm_name, self.final_norm = final_norm
        self.head_name, self.head = head
        # a position encoding that acts on the embedded rows (its on_embedding hook), mounted under its own name
        self.position_name, self.position = position if position is not None else (None, None)
        self.order: List[LayerRun] = list(order) if order is not None else [LayerRun(i) for i in range(len(self.layers))]
        self.ignorable_tensors = set(ignorable_tensors)
        self.vocab = self.embedding.vocab
        self.width = self.embedding.width
        # cache units: one per run that keeps its own cache
        self.run_unit: List[int] = []
        self.run_owns: List[bool] = []
        self.unit_needs: List[List[CacheNeed]] = []
        for i, run in enumerate(self.order):
            if not 0 <= run.layer < len(self.layers):
                raise ValueError(f"run {i} names layer {run.layer}, the model has {len(self.layers)}")
            if run.reads_cache_of is None:
                self.run_unit.append(len(self.unit_needs))
                self.run_owns.append(True)
                self.unit_needs.append(self.layers[run.layer][1].mixer.cache_needs())
            else:
                j = run.reads_cache_of
                if not 0 <= j < i or not self.run_owns[j]:
                    raise ValueError(f"run {i} reads the cache of run {j}, which must be an earlier run with a cache of its own")
                self.run_unit.append(self.run_unit[j])
                self.run_owns.append(False)

    # -- tensors ---------------------------------------------------------------
    def named_parts(self) -> Iterator[Tuple[str, Part]]:
        yield self.embedding_name, self.embedding
        if self.position is not None:
            yield self.position_name, self.position
        for prefix, block in self.layers:
            for name, part in block.parts():
                yield f"{prefix}.{name}", part
        yield self.final_norm_name, self.final_norm
        yield self.head_name, self.head

    def expected_tensors(self) -> Dict[str, TensorSpec]:
        out: Dict[str, TensorSpec] = {}
        for prefix, part in self.named_parts():
            for name, spec in part.tensor_specs().items():
                out[f"{prefix}.{name}"] = spec
        return out

    def kernel_variants(self, dtype: torch.dtype):
        seen = []
        for _, part in self.named_parts():
            for v in part.kernel_variants(dtype):
                if v not in seen:
                    seen.append(v)
        if ("sampling", ()) not in seen:
            seen.append(("sampling", ()))
        return seen

    def prepare(self, max_positions: int, device: torch.device) -> None:
        for _, block in self.layers:
            block.mixer.prepare(max_positions, device)
        if self.position is not None:
            self.position.prepare(max_positions, device)

    # -- the forward pass over the rows of a step -------------------------------
    def hidden(self, ctx, token_ids: torch.Tensor, all_rows_wanted: bool = False) -> torch.Tensor:
        """The residual rows after the last block.  all_rows_wanted: logits() will be asked for every row, so the last
        block may leave the final norm of its rows too (kept in ctx.final_normed for logits())."""
        ctx.final_normed = None
        x = ctx.buffer("model.residual", (token_ids.shape[0], self.width), torch.float32)
        self.embedding(token_ids, x)
        if self.position is not None:
            self.position.on_embedding(x, ctx)
        # A block may leave the next block's entry norm of its result beside the result (two sets of rows in turn).
        normed = None
        for i, run in enumerate(self.order):
            block = self.layers[run.layer][1]
            if not block.takes_normed:
                block.forward(x, ctx, self.run_unit[i], self.run_owns[i])
                normed = None
                continue
            last = i + 1 == len(self.order)
            nxt = None if last else self.layers[self.order[i + 1].layer][1]
            then = None
            if nxt is not None and nxt.takes_normed:
                then = (nxt.entry_norm, ctx.buffer(f"model.normed.{i & 1}", tuple(x.shape), ctx.dtype), nxt.mixer)
            elif last and all_rows_wanted:
                then = (self.final_norm, ctx.buffer(f"model.normed.{i & 1}", tuple(x.shape), ctx.dtype), self.head)
            left = block.forward(x, ctx, self.run_unit[i], self.run_owns[i], normed=normed, then=then)
            normed = (then[1] if left is True else left) if left else None     # True: the rows hold the norm
            if last and left:
                ctx.final_normed = normed
        return x

    def logits(self, ctx, x: torch.Tensor, rows: Optional[torch.Tensor], out: torch.Tensor) -> torch.Tensor:
        """Final norm and output head on the wanted rows of x (all rows if `rows` is None)."""
        if rows is None and getattr(ctx, "final_normed", None) is not None:
            return self.head(ctx.final_normed, out)         # the last block left the final norm of every row
        if rows is None and self.head.fuses_norm(self.final_norm, ctx):
            return self.head(x, out, norm=self.final_norm)
        xn = ctx.buffer("model.head_in", (out.shape[0], self.width), ctx.dtype)
        self.final_norm(x, xn, rows)
        return self.head(xn, out)
