"""What the parts see of one step: the rows' token ids, positions and sequences as
device arrays, the cache, and scratch buffers that keep their addresses (so that
a captured step can be replayed)."""
from __future__ import annotations

from typing import Dict, List, Optional, Sequence, Tuple

import numpy as np
import torch


class Workspace:
    """Named scratch buffers with room for `max_rows` rows each; a buffer is allocated
    at its first use and never moves afterwards."""

    def __init__(self, device: torch.device, max_rows: int):
        self.device = device
        self.max_rows = max_rows
        self._bufs: Dict[Tuple[str, int, torch.dtype], torch.Tensor] = {}
        self._retired: List[torch.Tensor] = []
        self._views: Dict[str, Tuple[tuple, torch.dtype, torch.Tensor]] = {}    # name -> the last (shape, dtype, view) handed out

    def get(self, name: str, shape: Sequence[int], dtype: torch.dtype) -> torch.Tensor:
        # the layers of a step ask for the same rows one after the other: the view made for the first serves the rest
        # (views keep no state of their own, and the buffer under them never moves)
        last = self._views.get(name)
        if last is not None and last[0] == shape and last[1] is dtype:
            return last[2]
        rows = int(shape[0])
        cols = 1
        for n in shape[1:]:
            cols *= int(n)
        if rows > self.max_rows:
            raise RuntimeError(f"workspace {name}: {rows} rows asked, room for {self.max_rows}")
        key = (name, cols, dtype)
        buf = self._bufs.get(key)
        if buf is None:
            buf = torch.empty((self.max_rows, cols), dtype=dtype, device=self.device)
            self._bufs[key] = buf
        view = buf[:rows].view(rows, *shape[1:]) if len(shape) > 1 else buf[:rows, 0]
        self._views[name] = (tuple(shape), dtype, view)
        return view

    def flat(self, name: str, n: int, dtype: torch.dtype, zero: bool = False) -> torch.Tensor:
        """A flat scratch buffer of at least n elements (zero-filled when made, if asked).  When a larger one
        is needed the old one is kept alive, because a captured step may still point at it."""
        key = ("flat:" + name, 0, dtype)
        buf = self._bufs.get(key)
        if buf is None or buf.numel() < n:
            if buf is not None:
                self._retired.append(buf)
            buf = (torch.zeros if zero else torch.empty)(n, dtype=dtype, device=self.device)
            self._bufs[key] = buf
        return buf

    def bytes(self) -> int:
        return sum(b.numel() * b.element_size() for b in self._bufs.values())


class StepContext:
    """Device arrays of a step (or of one piece of a step that was cut along its rows).

    token_ids, positions, tok_seq: one entry per row (int32); tok_seq is the index of the row's
    sequence in this step.  slots, start_pos, cu_q: one entry per sequence (cu_q one more): the
    sequence's slot, the length it had before this step, and the offset of its first row.
    The same numbers are kept on the host (`*_host`) for parts that plan launches.
    """

    def __init__(self, engine, n_seq: int, n_tokens: int, arrays: Dict[str, torch.Tensor], host: Dict[str, np.ndarray]):
        self.engine = engine
        self.cache = engine.cache
        self.dtype: torch.dtype = engine.dtype
        self.device: torch.device = engine.device
        self.n_seq, self.n_tokens = n_seq, n_tokens
        self.token_ids = arrays["token_ids"]
        self.positions = arrays["positions"]
        self.tok_seq = arrays["tok_seq"]
        self.slots = arrays["slots"]
        self.start_pos = arrays["start_pos"]
        self.cu_q = arrays["cu_q"]
        self.arrays = arrays
        self.host = host
        q_lens = host["q_lens"]
        self.max_q_len = int(q_lens.max()) if n_seq else 0
        self.is_decode = bool(n_seq) and self.max_q_len == 1
        self.max_kv_len = int((host["start_pos"] + q_lens).max()) if n_seq else 0

        #: pages any sequence of this step may hold (a captured step must allow for the whole context)
        self.max_pages_used: Optional[int] = None
        #: steps of single tokens: for each storage group of the cache, the sequences' page-table rows in the order of
        #: the step ([>= n_seq, the table's width], row i = the row of slots[i]), kept current by the engine
        self.seq_pages: Dict[int, torch.Tensor] = {}

    def buffer(self, name: str, shape: Sequence[int], dtype: torch.dtype) -> torch.Tensor:
        return self.engine.workspace.get(name, shape, dtype)

    def scratch(self, name: str, n: int, dtype: torch.dtype, zero: bool = False) -> torch.Tensor:
        return self.engine.workspace.flat(name, n, dtype, zero)
