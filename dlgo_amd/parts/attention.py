"""The attention mixer: grouped-query attention over the paged cache.

Per token (computerex/dlgo, models/llm/forward.go:207-290): q, k, v projections
without bias (:224), rotation of each q and k head (:246-252), keys (rotated) and
values stored at the token's position (:257), then for query head h the softmax
over the scores against keys 0..p of KV head h // (H/KV), scaled by 1/sqrt(hd)
(:258-278), and the output projection (:286).  The three projections are one
matrix product against the fused [q|k|v] rows, the rotation and the cache write
are one kernel, and the output projection adds into the float32 residual stream.

The mixer's sizes are its parameters; `window` limits each token to the last
`window` keys (layers/gqa.go:98-132).  A run of the layer that reads another
run's cache computes queries only and stores nothing.

Two options that the reference applies when a layer has the tensors for them
(models/llm/forward.go:227-244), both between projection and rotation: biases of
the projections (`bias`; `out_bias` for the output projection's), and an RMSNorm
of every q and k head over the head's own elements (`qk_norm_eps`).  A layer
without them launches nothing for them; a layer with them takes the separate
rotation kernel, since the fused ones read the product's result as it is.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

from ..kernels import ops
from .base import CacheNeed, Part, TensorSpec, check_inner, stored
from .norm import RMSNorm
from .position import PositionEncoding


class Mixer(Part):
    """Interface of a sequence mixer.

    cache_needs(): what one run of the layer keeps per sequence.
    forward(xn, ctx, unit, residual, owns_cache): xn are the normed rows of the step (run dtype, [T, width]);
    the result is added into `residual` (float32 [T, width]).  `unit` is the cache unit this run reads;
    `owns_cache` is False when the unit belongs to another run (then nothing is stored).
    A mixer with state must treat the rows of a sequence in order: ctx.cu_q gives each sequence's rows.

    A mixer that sets `leaves_norm` also takes then=(norm part, rows) or (norm part, rows, the part that will read
    them): "if it costs you nothing, leave that norm of the residual rows as they are after you in `rows`", and returns
    True if it did (the block then skips the norm), or, if the reading part takes_unscaled(), a kernels.ops.UnscaledNorm
    that describes what it left instead (the block hands that to the reading part in place of the rows).
    """
    leaves_norm = False

    def cache_needs(self) -> List[CacheNeed]:
        return []

    def prepare(self, max_positions: int, device: torch.device) -> None:
        pass

    def fuses_norm(self, norm, ctx) -> bool:
        """True if, for this step, the mixer would rather be given the float32 residual rows and the norm
        part (forward(x, ..., norm=norm)) than the normed rows."""
        return False

    def forward(self, xn: torch.Tensor, ctx, unit: int, residual: torch.Tensor, owns_cache: bool = True, norm=None) -> None:
        raise NotImplementedError


class Attention(Mixer):
    leaves_norm = True

    def __init__(self, width: int, n_heads: int, n_kv_heads: int, head_dim: int, position: PositionEncoding,
                 window: Optional[int] = None, scale: Optional[float] = None, bias: bool = False, out_bias: bool = False,
                 qk_norm_eps: Optional[float] = None):
        if n_heads % n_kv_heads:
            raise ValueError(f"attention: {n_heads} heads are not a multiple of {n_kv_heads} kv heads")
        if head_dim % 16:
            raise ValueError(f"attention: head size {head_dim} is not a multiple of 16 (the kernels take steps of 16)")
        self.width, self.n_heads, self.n_kv_heads, self.head_dim = width, n_heads, n_kv_heads, head_dim
        self.q_dim, self.kv_dim = n_heads * head_dim, n_kv_heads * head_dim
        self.position = position
        self.window = window
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(head_dim)
        self.bias, self.out_bias = bool(bias), bool(out_bias)
        self.qk_norm_eps = None if qk_norm_eps is None else float(qk_norm_eps)
        self.w_qkv: Optional[torch.Tensor] = None
        self.w_o: Optional[torch.Tensor] = None
        self.b_qkv: Optional[torch.Tensor] = None
        self.b_o: Optional[torch.Tensor] = None
        self.q_norm: Optional[torch.Tensor] = None
        self.k_norm: Optional[torch.Tensor] = None

    @property
    def kernel_modules(self):
        extra = ("rowwise",) if self.bias or self.out_bias or self.qk_norm_eps is not None else ()
        return ("gemm", "gemm_rows", "rope_kv") + extra

    def tensor_specs(self) -> Dict[str, TensorSpec]:
        specs = {
            "q_proj.weight": TensorSpec((self.q_dim, self.width)),
            "k_proj.weight": TensorSpec((self.kv_dim, self.width)),
            "v_proj.weight": TensorSpec((self.kv_dim, self.width)),
            "o_proj.weight": TensorSpec((self.width, self.q_dim)),
        }
        if self.bias:
            specs.update({"q_proj.bias": TensorSpec((self.q_dim,), kind="vector", init="normal"),
                          "k_proj.bias": TensorSpec((self.kv_dim,), kind="vector", init="normal"),
                          "v_proj.bias": TensorSpec((self.kv_dim,), kind="vector", init="normal")})
        if self.out_bias:
            specs["o_proj.bias"] = TensorSpec((self.width,), kind="vector", init="normal")
        if self.qk_norm_eps is not None:
            specs.update({"q_norm.weight": TensorSpec((self.head_dim,), kind="vector", init="ones"),
                          "k_norm.weight": TensorSpec((self.head_dim,), kind="vector", init="ones")})
        return specs

    MAX_HEAD_DIM = 512       # the attention kernels are compiled per head size, up to this one

    def check(self, dtype) -> None:
        check_inner("attention", (("width", self.width), ("heads * head size", self.q_dim)), dtype)
        if self.head_dim > self.MAX_HEAD_DIM:
            raise ValueError(f"attention: head size {self.head_dim} is beyond the kernels' largest, {self.MAX_HEAD_DIM}")

    def kernel_variants(self, dtype):
        from ..kernels.build import variant
        return tuple(variant(m, dtype) for m in self.kernel_modules) + (variant("attention", dtype, (("HEAD_DIM", self.head_dim),)),)

    def cache_needs(self) -> List[CacheNeed]:
        return [CacheNeed(kind="kv", kv_heads=self.n_kv_heads, head_dim=self.head_dim, window=self.window)]

    def prepare(self, max_positions: int, device: torch.device) -> None:
        self.position.prepare(max_positions, device)

    def load(self, tensors, device, dtype) -> None:
        spec = self.tensor_specs()
        fused = torch.cat([tensors["q_proj.weight"], tensors["k_proj.weight"], tensors["v_proj.weight"]], dim=0)
        self.w_qkv = stored(fused, spec["q_proj.weight"], device, dtype)
        self.w_o = stored(tensors["o_proj.weight"], spec["o_proj.weight"], device, dtype)
        if self.bias:
            fused_b = torch.cat([tensors["q_proj.bias"].float(), tensors["k_proj.bias"].float(), tensors["v_proj.bias"].float()])
            self.b_qkv = stored(fused_b, spec["q_proj.bias"], device, dtype)
        if self.out_bias:
            self.b_o = stored(tensors["o_proj.bias"], spec["o_proj.bias"], device, dtype)
        if self.qk_norm_eps is not None:
            self.q_norm = stored(tensors["q_norm.weight"], spec["q_norm.weight"], device, dtype)
            self.k_norm = stored(tensors["k_norm.weight"], spec["k_norm.weight"], device, dtype)

    @property
    def _between(self) -> bool:
        """Something stands between the projections and the rotation."""
        return self.bias or self.qk_norm_eps is not None

    def fuses_norm(self, norm, ctx) -> bool:
        return isinstance(norm, RMSNorm) and ops.fused_norm_pays(self.w_qkv, ctx.n_tokens)

    def takes_unscaled(self, ctx) -> bool:
        return ops.can_take_unscaled(self.w_qkv, ctx.n_tokens)

    def forward(self, xn, ctx, unit, residual, owns_cache=True, norm=None, then=None):
        t = residual.shape[0]
        n_kv = self.n_kv_heads if owns_cache else 0
        cols = self.q_dim + 2 * n_kv * self.head_dim
        qkv = ctx.buffer("attention.qkv", (t, self.q_dim + 2 * self.kv_dim), ctx.dtype)
        split = ctx.scratch("gemm.split", ops.GEMM_SPLIT_FLOATS, torch.float32)
        kv = ctx.cache.kv_view(unit)
        rot = self.position.rotation()
        # a step of single tokens: the attention kernel rotates and stores by itself; else a kernel of its own does
        fused = not self._between and ops.attention_fuses_rotation(ctx.dtype, self.head_dim, self.n_heads // self.n_kv_heads,
                                                                   ctx.max_q_len, rot.width if rot else 0, ctx.n_seq, self.n_kv_heads)
        unsummed = None
        if isinstance(xn, ops.UnscaledNorm):   # the norm's factor is applied to the product's sums
            ops.gemm_scaled(self.w_qkv[:cols], xn, qkv[:, :cols])
        elif norm is not None:    # xn are the float32 residual rows: the norm rides in the product
            ops.gemm_rmsnorm(self.w_qkv[:cols], xn, norm.weight, norm.eps, qkv[:, :cols])
        else:
            # a product that shares k out over blocks leaves its runs to the rotation kernel, which adds them up as it reads
            if not fused and not self._between and ops.rope_takes_unsummed(ctx.dtype, self.head_dim, rot.width if rot else 0):
                unsummed = ops.gemm_runs(self.w_qkv[:cols], xn, split)
            if unsummed is None:
                ops.gemm(self.w_qkv[:cols], xn, qkv[:, :cols], scratch=split)
        if self.bias:
            ops.bias_add(qkv[:, :cols], self.b_qkv[:cols])
        if self.qk_norm_eps is not None:
            ops.head_rmsnorm(qkv, 0, self.n_heads, self.head_dim, self.q_norm, self.qk_norm_eps)
            if n_kv:
                ops.head_rmsnorm(qkv, self.q_dim, n_kv, self.head_dim, self.k_norm, self.qk_norm_eps)
        if not fused:
            ops.rope_kv(qkv, self.n_heads, n_kv, self.head_dim, rot.width if rot else 0, rot.interleaved if rot else False,
                        rot.cos if rot else None, rot.sin if rot else None, ctx.positions,
                        ctx.tok_seq, ctx.slots, kv.page_table, kv.cache, kv.page_stride, kv.v_off, write_kv=owns_cache,
                        unsummed=unsummed, single_tokens=ctx.max_q_len == 1,
                        seq_pages=getattr(ctx, "seq_pages", {}).get(kv.group) if ctx.max_q_len == 1 else None)
        out = ctx.buffer("attention.out", (t, self.q_dim), ctx.dtype)
        self.attend(qkv, out, ctx, kv, rotation=(rot.cos, rot.sin, rot.width, rot.interleaved) if fused and rot else None,
                    new_kv=fused and owns_cache)
        if self.out_bias:        # the bias goes into the residual after the product: no norm of it can be left on the way
            ops.gemm(self.w_o, out, residual, ops.EPI_ACCUM_F32, scratch=split)
            ops.bias_add(residual, self.b_o)
            return False
        if then is not None and isinstance(then[0], RMSNorm):
            # the norm left unscaled by a streamed product (few rows); else written whole by the sum of a product whose k
            # was shared out; else left unscaled by a tiled product (many rows); else not at all
            unscaled_ok = len(then) > 2 and then[2] is not None and then[2].takes_unscaled(ctx)

            def leave():
                shares = ctx.scratch("attention.norm_shares", t * ((self.width + 7) // 8), torch.float32)
                return ops.gemm_accum_leave_norm(self.w_o, out, residual, then[0].weight, then[0].eps, then[1], shares)
            if unscaled_ok and ops.streams_few_rows(self.w_o, t, ops.ROLE_LEAVES_NORM):
                return leave()
            if ops.gemm_accum_then_norm(self.w_o, out, residual, split, then[0].weight, then[0].eps, then[1]):
                return True
            if unscaled_ok and ops.can_leave_unscaled(self.w_o, t):
                return leave()
        ops.gemm(self.w_o, out, residual, ops.EPI_ACCUM_F32, scratch=split)
        return False

    def attend(self, q, out, ctx, kv, rotation=None, new_kv=False) -> None:
        """Attention of the step's (rotated) query rows over the cache; the kernel is chosen by the
        step's shape and the run dtype, the arithmetic is the same."""
        ops.attention(q, out, self.n_heads, self.n_kv_heads, self.head_dim, ctx.positions, ctx.tok_seq, ctx.slots,
                      kv.page_table, kv.cache, kv.page_stride, kv.v_off, ctx.host["q_lens"], ctx.host["start_pos"],
                      window=self.window or 0, scale=self.scale, cu_q=ctx.cu_q, start_pos_dev=ctx.start_pos,
                      scratch=lambda n: ctx.scratch("attention.partials", n, torch.float32),
                      max_pages_used=ctx.max_pages_used, rotation=rotation, new_kv=new_kv,
                      seq_pages=getattr(ctx, "seq_pages", {}).get(kv.group) if ctx.max_q_len == 1 else None)
