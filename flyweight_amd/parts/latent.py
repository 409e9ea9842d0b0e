"""Attention over a cached latent, without positions or with a rotated part beside the latent.

The query passes a low-rank map with a norm in its middle: c_q = rms(W_dq h) * w_q, q = W_uq c_q
(heads of ``head_dim`` channels). Keys and values of every head are linear maps of one latent per
token, c = rms(W_dkv h) * w_kv (``kv_rank`` channels): k_i = W_uk,i c, v_i = W_uv,i c (values of
``v_head_dim`` channels). Scores q_i . k_i * softmax_scale over every earlier token and the row itself,
softmax in float32; the heads side by side are multiplied by sigmoid(W_g h) and pass W_o.

Only c is cached, and the two maps move to the query's side of the products: q_i . (W_uk,i c) =
(W_uk,i^T q_i) . c, and sum_j p_j (W_uv,i c_j) = W_uv,i (sum_j p_j c_j). The paged attention kernels then
see ``num_heads`` query heads of ``kv_rank`` channels over ONE key/value head whose keys and values are
both c (each in the layout its product reduces over), whatever the number of heads; the gate rides in
the epilogue of the map back to the values' size. An RMS norm here is x / sqrt(mean(x^2) + eps).

``rot_dim`` r > 0 gives positions to the scores: a query head has ``head_dim`` channels for the latent's keys and r more
that are rotated; W_dkv has r more rows whose output (not normed) is one rotated key part per token that all heads
share, and the score is q_plain . k_plain + q_rot . k_rot. The cache's one key head then holds [c | rotated part]
(``kv_rank`` + r channels) and its value head c; a query is [W_uk^T q_plain | rotated q_rot] and nothing else changes.
``position`` names the rotation (its tables are made for r channels). ``output_gate`` False: no gate, no W_g.
"""

from __future__ import annotations

from typing import Dict

import torch

from ..cache.needs import PagedKV
from ..config.spec import ConfigError, PartSpec
from ..kernels import ops
from ..weights.loader import TensorDecl
from .attention import QueryTileArrays
from .base import Mixer, build_part, register_mixer
from .linear import Linear
from .norm import LazyNorm

_DEFAULT_NAMES = {"dq": "dq", "dq_norm": "dq.norm", "uq": "uq", "dkv": "dkv", "dkv_norm": "dkv.norm", "uk": "uk", "uv": "uv",
                  "g": "g", "o": "o"}


@register_mixer("latent_attention")
class LatentAttention(QueryTileArrays, Mixer):
    graph_safe = True

    def __init__(self, spec):
        super().__init__(spec)
        self.hidden = int(spec["hidden_size"])
        self.num_heads = int(spec["num_heads"])
        self.head_dim = int(spec["head_dim"])
        self.v_head_dim = int(spec.get("v_head_dim") or self.head_dim)
        self.q_rank = int(spec["q_rank"])
        self.kv_rank = int(spec["kv_rank"])
        self.eps = float(spec["norm_eps"])
        self.scale = float(spec.get("softmax_scale", self.head_dim ** -0.5))
        self.gated = bool(spec.get("output_gate", True))
        self.rot_dim = int(spec.get("rot_dim") or 0)
        self.position = build_part("position", spec["position"]) if self.rot_dim else None
        self.names = {**_DEFAULT_NAMES, **dict(spec.get("names", {}))}
        # the norm in the middle of the query's map is a norm part: the product behind it may take it into its own kernel
        self.q_norm = build_part("norm", PartSpec("rmsnorm", {"size": self.q_rank, "eps": self.eps, "tensor": self._name("dq_norm")}))
        if not 1 <= self.kv_rank + self.rot_dim <= ops.MAX_PLAIN_HEAD_DIM:     # (beyond the matrix-core kernels' 256 channels the plain kernel serves)
            raise ConfigError(f"a latent of {self.kv_rank} + {self.rot_dim} channels exceeds the attention kernels' limit of {ops.MAX_PLAIN_HEAD_DIM}")
        self.turned = int(getattr(self.position, "rotary_dim", 0)) if self.rot_dim else 0
        if self.rot_dim and (self.rot_dim % 2 or self.turned % 2 or self.turned > self.rot_dim or
                             (self.turned and not getattr(self.position, "interleaved", False))):
            raise ConfigError("the rotated part of a latent's keys is even in size and pairs neighbouring channels, its first ones or all")
        if min(self.num_heads, self.head_dim, self.v_head_dim, self.q_rank) < 1:
            raise ConfigError("latent attention: every size must be positive")

    @property
    def key_dim(self) -> int:
        """Channels of a cached key: the latent and the rotated part behind it."""
        return self.kv_rank + self.rot_dim

    def cache_need(self):
        return PagedKV(1, self.key_dim, None, self.kv_rank if self.rot_dim else None)

    def _name(self, which: str) -> str:
        return self.prefix + self.names[which]

    def tensors(self) -> Dict[str, TensorDecl]:
        D, H, d, dv, rq, rk, dr = self.hidden, self.num_heads, self.head_dim, self.v_head_dim, self.q_rank, self.kv_rank, self.rot_dim
        declared = {
            self._name("dq"): TensorDecl((rq, D)), **self.q_norm.tensors(),
            self._name("uq"): TensorDecl((H * (d + dr), rq)),
            self._name("dkv"): TensorDecl((rk + dr, D)), self._name("dkv_norm"): TensorDecl((rk,), "vector", "norm"),
            self._name("uk"): TensorDecl((H * d, rk)), self._name("uv"): TensorDecl((H * dv, rk)),
            self._name("o"): TensorDecl((D, H * dv)),
        }
        if self.gated:
            declared[self._name("g")] = TensorDecl((H * dv, D))
        return declared

    def bind(self, tensors, dtype, device) -> None:
        super().bind(tensors, dtype, device)
        self.q_norm.bind(tensors, dtype, device)
        if self.position is not None:
            self.position.bind(tensors, dtype, device)
        t = {which: tensors[self._name(which)] for which in self.names if self._name(which) in tensors}
        H, d, dv, rk = self.num_heads, self.head_dim, self.v_head_dim, self.kv_rank
        # what reads h: the query's inner map, and the latent's with the gate behind it in one operand
        # (float32 sums out: the norms and the sigmoid read them as they are)
        self.down_q = Linear(t["dq"])
        self.down_kv = Linear(torch.cat([t["dkv"], t["g"]], dim=0) if self.gated else t["dkv"])
        self.up_q = Linear(t["uq"])
        # per head: the keys' map transposed (it is applied to the query), the values' map as it is
        self.uk_t = t["uk"].reshape(H, d, rk).transpose(1, 2).contiguous()       # [H][rk][d]
        self.uv = t["uv"].reshape(H, dv, rk).contiguous()                        # [H][dv][rk]
        self.out = Linear(t["o"])
        self.kv_norm_weight = t["dkv_norm"]

    def uses_query_tiles(self) -> bool:
        return getattr(self, "dtype", None) == torch.bfloat16 and ops.attention_is_tiled(self.kv_rank) and ops.attention_is_tiled(self.key_dim)

    def mixing_flops(self, rows: int, keys_before: int = 0) -> int:
        """Scores and weighted sums over the latent for rows that follow ``keys_before`` cached tokens,
        and the two maps per head around them."""
        pairs = rows * keys_before + rows * (rows + 1) // 2
        return 2 * self.num_heads * (self.key_dim + self.kv_rank) * pairs + 2 * rows * self.num_heads * self.kv_rank * (self.head_dim + self.v_head_dim)

    def heads_output(self, h, ctx, cache) -> torch.Tensor:
        """The gated heads [rows, heads * v_head_dim] in the activation dtype; the step's latents join the cache."""
        down = self.down_kv.forward(h, out_dtype=torch.float32)
        cos, sin = ctx.position_tables(self.position) if self.turned else (None, None)
        if cache.writes:
            ops.latent_norm_write(down[:, :self.key_dim], self.kv_norm_weight, self.eps, cache.k_pages, cache.v_pages,
                                  cache.block_table, ctx.row_seg, ctx.row_pos, rot=self.rot_dim, cos=cos, sin=sin, turn=self.turned)
        # (for a few rows of a bfloat16 model the norm runs inside the product that reads it)
        q = self.up_q.forward(LazyNorm(self.q_norm, self.down_q.forward(h, out_dtype=torch.float32), ctx))
        if self.rot_dim:
            # a query against the cached keys: [W_uk^T q_plain | q_rot turned], head by head
            q_latent = torch.empty((q.shape[0], self.num_heads * self.key_dim), dtype=self.dtype, device=q.device)
            ops.head_linear(q, self.uk_t, self.dtype, in_head=self.head_dim + self.rot_dim, out=q_latent, out_head=self.key_dim)
            ops.rotate_place(q, self.num_heads, self.head_dim, self.rot_dim, cos, sin, q_latent, self.kv_rank, turn=self.turned)
        else:
            q_latent = ops.head_linear(q, self.uk_t, self.dtype)                      # [rows, H * rk]
        own = ctx.step_arrays(self) if self.step_arrays_key() is not None else {}
        mixed = ops.attention(q_latent, self.num_heads, 1, self.key_dim, cache.k_pages, cache.v_pages, cache.block_table, ctx,
                              self.scale, 0, tile_seg=own.get("tile_seg"), tile_row0=own.get("tile_row0"),
                              decode_work=own.get("decode_work"), v_dim=self.kv_rank)
        gate = down[:, self.key_dim:] if self.gated else None
        return ops.head_linear(mixed, self.uv, self.dtype, gate=gate)

    def output(self, h, ctx, cache) -> torch.Tensor:
        return self.out.forward(self.heads_output(h, ctx, cache), out_dtype=torch.float32)

    def forward(self, h, residual, ctx, cache):
        return self.out.accumulate(self.heads_output(h, ctx, cache), residual, then=getattr(ctx, "upcoming_norm", None))
