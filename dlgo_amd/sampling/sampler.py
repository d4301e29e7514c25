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
    def __init__(self, vocab: int, device, max_rows: int = 256):
        self.vocab = vocab
        self.device = torch.device(device)
        self.max_rows = max_rows
        self._out = torch.empty(max_rows, dtype=torch.int32, device=self.device)
        self._work: Optional[torch.Tensor] = None
        self._e: Optional[torch.Tensor] = None

    def _grow(self, rows: int) -> None:
        if rows > self._out.shape[0]:
            self._out = torch.empty(rows, dtype=torch.int32, device=self.device)
            self._work = self._e = None

    def choose(self, logits: torch.Tensor, configs: Sequence[SamplerConfig], uniforms: Sequence[float],
               recent: Optional[Sequence[Sequence[int]]] = None) -> List[int]:
        """logits [rows, vocab] float32 on the device -> one token id per row (host list)."""
        n = logits.shape[0]
        if n != len(configs) or n != len(uniforms):
            raise ValueError("sampler: one configuration and one uniform number per row")
        self._grow(n)
        out = self._out[:n]
        if all(c.greedy for c in configs):
            ops.argmax(logits, out)
            return out.tolist()
        if self._work is None:
            rows = self._out.shape[0]
            self._work = torch.empty((rows, self.vocab), dtype=torch.float32, device=self.device)
            self._e = torch.empty((rows, self.vocab), dtype=torch.float32, device=self.device)
        f = np.zeros((5, n), dtype=np.float32)
        k = np.zeros(n, dtype=np.int32)
        for i, c in enumerate(configs):
            f[0, i], f[1, i], f[2, i], f[3, i], f[4, i] = c.temperature, c.top_p, c.min_p, c.repetition_penalty, uniforms[i]
            k[i] = c.top_k
        fd = torch.from_numpy(f).to(self.device)
        kd = torch.from_numpy(k).to(self.device)
        rec = None
        if recent is not None and any(c.repetition_penalty > 1.0 and not c.greedy for c in configs):
            r = np.full((n, RECENT), -1, dtype=np.int32)
            for i, toks in enumerate(recent):
                toks = list(toks)[-RECENT:]
                r[i, :len(toks)] = toks
            rec = torch.from_numpy(r).to(self.device)
        ops.sample(logits, self._work, self._e, fd[0], kd, fd[1], fd[2], fd[3], rec, fd[4], out)
        return out.tolist()
