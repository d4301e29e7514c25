"""Next tokens from logits on the device: argmax when every row is greedy, else
the sampling kernel with each row's own options."""
from __future__ import annotations

from typing import List, Optional, Sequence

import numpy as np
import torch

from ..kernels import ops
from .options import SamplerConfig

RECENT = 64   # tokens the repetition penalty looks back on (models/llm/generate.go:361-365)


class Sampler:
    #: the tokens a request has been given are also kept on the device (start(), and keys= of the choose calls), so
    #: that the repetition penalty does not need them back from the host before the next choice
    keeps_recent = True

    def __init__(self, vocab: int, device, max_rows: int = 256):
        self.vocab = vocab
        self.device = torch.device(device)
        self.max_rows = max_rows
        self._out = torch.empty(max_rows, dtype=torch.int32, device=self.device)
        self._pinned = [torch.empty(max_rows, dtype=torch.int32, pin_memory=True) for _ in range(4)]
        self._pin_next = 0
        self._work: Optional[torch.Tensor] = None
        # the rows' options go up in one copy from pinned memory that does not wait for the device: a copy from
        # ordinary memory would hold the host until the step queued before it is done, and the step after it with it
        self._staging: List[tuple] = []                 # (pinned int32 buffer, event of the copy that last read it)
        self._staging_next = 0
        self._options: Optional[torch.Tensor] = None    # the device's copy: 7 rows of int32/float32 bits
        self._rings: Optional[torch.Tensor] = None      # [keys, RECENT] last tokens chosen per key
        self._counts: Optional[torch.Tensor] = None     # [keys] tokens chosen so far per key

    def start(self, keys: Sequence[int]) -> None:
        """Requests begin under these keys (any small integers that stay with a request, such as its slot): what the
        device remembers of earlier requests under them is forgotten."""
        need = max(keys) + 1 if len(keys) else 0
        if self._counts is None or self._counts.shape[0] < need:
            size = max(need, 2 * (self._counts.shape[0] if self._counts is not None else 0), self.max_rows)
            counts = torch.zeros(size, dtype=torch.int32, device=self.device)
            rings = torch.full((size, RECENT), -1, dtype=torch.int32, device=self.device)
            if self._counts is not None:
                counts[:self._counts.shape[0]] = self._counts
                rings[:self._rings.shape[0]] = self._rings
            self._counts, self._rings = counts, rings
        if len(keys):
            self._counts[torch.as_tensor(list(keys), dtype=torch.long)] = 0

    def _upload(self, f: np.ndarray, k: np.ndarray):
        """f [5, n] float32 and k [2, n] int32 -> their device copies, through one pinned buffer and one copy that the
        host does not wait for."""
        n = f.shape[1]
        if not self._staging:
            self._staging = [(torch.empty(7 * max(n, self.max_rows), dtype=torch.int32, pin_memory=True), None) for _ in range(4)]
        i = self._staging_next
        self._staging_next = (i + 1) % len(self._staging)
        buf, ev = self._staging[i]
        if ev is not None:
            ev.synchronize()
        if buf.numel() < 7 * n:
            buf = torch.empty(14 * n, dtype=torch.int32, pin_memory=True)
        hv = buf.numpy()
        hv[:5 * n] = f.reshape(-1).view(np.int32)
        hv[5 * n:7 * n] = k.reshape(-1)
        if self._options is None or self._options.numel() < 7 * n:
            self._options = torch.empty(14 * n, dtype=torch.int32, device=self.device)
        dev = self._options[:7 * n]
        dev.copy_(buf[:7 * n], non_blocking=True)
        ev = torch.cuda.Event()
        ev.record()
        self._staging[i] = (buf, ev)
        return dev[:5 * n].view(torch.float32).view(5, n), dev[5 * n:].view(2, n)

    def _grow(self, rows: int) -> None:
        if rows > self._out.shape[0]:
            self._out = torch.empty(rows, dtype=torch.int32, device=self.device)
            self._work = None

    def choose(self, logits: torch.Tensor, configs: Sequence[SamplerConfig], uniforms: Sequence[float],
               recent: Optional[Sequence[Sequence[int]]] = None) -> List[int]:
        """logits [rows, vocab] float32 on the device -> one token id per row (host list)."""
        return self.choose_device(logits, configs, uniforms, recent).tolist()

    def choose_async(self, logits: torch.Tensor, configs: Sequence[SamplerConfig], uniforms: Sequence[float],
                     recent: Optional[Sequence[Sequence[int]]] = None, keys: Optional[Sequence[int]] = None):
        """The ids as a device tensor (valid until the next call) and a function that waits for them and
        returns them as a host list; work can be queued behind the choice before the ids are awaited.
        keys (instead of recent): each row's key as given to start(); the recent tokens are the device's own record."""
        out = self.choose_device(logits, configs, uniforms, recent, keys)
        n = out.shape[0]
        i = self._pin_next
        self._pin_next = (i + 1) % len(self._pinned)
        host = self._pinned[i]
        if host.shape[0] < n:
            host = self._pinned[i] = torch.empty(max(n, 2 * host.shape[0]), dtype=torch.int32, pin_memory=True)
        host[:n].copy_(out, non_blocking=True)
        event = torch.cuda.Event()
        event.record()

        def wait() -> List[int]:
            event.synchronize()
            return host[:n].tolist()
        return out, wait

    def needs_recent(self, configs: Sequence[SamplerConfig]) -> bool:
        """True if a row's choice depends on the tokens generated so far (the repetition penalty)."""
        return any(c.repetition_penalty > 1.0 and not c.greedy for c in configs)

    def choose_device(self, logits: torch.Tensor, configs: Sequence[SamplerConfig], uniforms: Sequence[float],
                      recent: Optional[Sequence[Sequence[int]]] = None, keys: Optional[Sequence[int]] = None) -> torch.Tensor:
        """logits [rows, vocab] float32 on the device -> int32 ids on the device (overwritten by the next call)."""
        n = logits.shape[0]
        if n != len(configs) or n != len(uniforms):
            raise ValueError("sampler: one configuration and one uniform number per row")
        self._grow(n)
        out = self._out[:n]
        if all(c.greedy for c in configs):
            ops.argmax(logits, out)
            return out
        if self._work is None:
            rows = self._out.shape[0]
            self._work = torch.empty((rows, self.vocab), dtype=torch.float32, device=self.device)
        f = np.zeros((5, n), dtype=np.float32)
        k = np.zeros((2, n), dtype=np.int32)        # top-k, and the row's key if the device keeps the recent tokens
        for i, c in enumerate(configs):
            f[0, i], f[1, i], f[2, i], f[3, i], f[4, i] = c.temperature, c.top_p, c.min_p, c.repetition_penalty, uniforms[i]
            k[0, i] = c.top_k
        penalised = any(c.repetition_penalty > 1.0 and not c.greedy for c in configs)
        rings = keys is not None and recent is None
        if rings:
            if self._counts is None or max(keys) >= self._counts.shape[0]:
                raise ValueError("sampler: keys that start() was never given")
            k[1] = np.asarray(keys, dtype=np.int32)
        fd, kd = self._upload(f, k)
        # rows that several blocks share: a top-k of up to 1,024, or neither top-k nor top-p; without one, two kernels need not be
        # launched (a hint only: which rows those kernels take they decide themselves, from the options on the device)
        dealt_rows = any(not c.greedy and (1 <= c.top_k <= 1024 or (not 0 < c.top_k < self.vocab and c.top_p >= 1.0))
                         for c in configs)
        if rings:       # every choice is recorded, penalty or not: a later row of the request may have one
            ops.sample(logits, self._work, fd[0], kd[0], fd[1], fd[2], fd[3], self._rings, fd[4], out,
                       recent_rows=kd[1], counts=self._counts, dealt_rows=dealt_rows)
            return out
        rec = None
        if recent is not None and penalised:
            r = np.full((n, RECENT), -1, dtype=np.int32)
            for i, toks in enumerate(recent):
                toks = list(toks)[-RECENT:]
                r[i, :len(toks)] = toks
            rec = torch.from_numpy(r).to(self.device)
        ops.sample(logits, self._work, fd[0], kd[0], fd[1], fd[2], fd[3], rec, fd[4], out, dealt_rows=dealt_rows)
        return out
