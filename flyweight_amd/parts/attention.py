"""Grouped-query attention over the paged cache.

q = W_q h, k = W_k h, v = W_v h; optional per-head RMS norm of q and k (one weight of
head_dim shared by all heads); position encoding on q and k; k and v appended to the
cache; scores q.k * softmax_scale (1 / sqrt(head_dim) unless given) over the cached keys the row
may see (causal, optionally only the last ``window``: itself and the window - 1 before it; with
``chunk`` only those of the row's own chunk of that many positions, chunks counted from position 0 of
the sequence), optionally capped softly (``score_softcap`` c: c tanh(score / c)), softmax in float32, weighted sum of values; out = W_o o.
Beside a window ``keep_first`` n keeps the first n keys of the sequence seen wherever the window stands
(row i sees key j <= i if i - j < window or j < n). ``sink`` gives every head a learned number s (tensor
``names["sink"]``, [heads]) whose exp(s) joins the softmax's denominator: a term with no key and no value, not
scaled. ``shared_kv``: the layer has no key and value projections; it reads the cache entry of another layer
(the schedule names it and says that this layer does not write it), with its own queries and mask. Values may have a size of their own
(``v_head_dim``); the output of a head has that size.
``values`` "keys": there is no W_v, a token's value is its key as it stands before the per-head norm (behind the
convolution, where there is one). ``qk_conv`` L: a short causal convolution of L taps per channel over time on q and k,
directly behind their projections (tensors ``names["q_conv"]``, ``names["k_conv"]``, [channels, L], the last column the
current token's; the request's slot keeps the last L - 1 projected rows). ``qk_bias``: biases on the q and k
projections alone (``names["q_bias"]``, ``names["k_bias"]``). ``sink`` "unit": the denominator's extra term is exp(0) = 1
for every head, nothing learned. ``distance_slope_exponent`` e: slope_h * (i - j) is taken off the score of row i and
key j behind the cap, slope_h = 2^(-e (h + 1) / heads). ``query_temperature`` (coef, every): the normed queries of
position p are multiplied by 1 + coef ln(floor((p + 1) / every) + 1).
Query head i reads kv head i // (num_heads / num_kv_heads). Formulas as the reference's
LFM2 attention branch computes them (native/src/v2_runtime.cpp:28429-28478).
"""

from __future__ import annotations

from typing import Dict

import numpy as np
import torch

from ..cache.needs import FixedState, PagedKV
from ..config.spec import ConfigError, PartSpec
from ..kernels import ops
from ..weights.loader import TensorDecl
from .base import Mixer, build_part, register_mixer
from .linear import Linear

_DEFAULT_NAMES = {"q": "q_proj", "k": "k_proj", "v": "v_proj", "o": "o_proj", "q_norm": "q_norm", "k_norm": "k_norm", "sink": "sink",
                  "q_bias": "q_proj.bias", "k_bias": "k_proj.bias", "q_conv": "q_conv", "k_conv": "k_conv"}


class QueryTileArrays:
    """What a mixer that runs the matrix-core attention kernels over the paged cache asks of a step's upload
    (``Part.step_arrays``). The prompt kernel works on tiles of up to 64 rows of one segment: which tiles
    there are, and in which order workgroups take them. The split-key decode kernel shares a step's work out
    over the chip by the number of runs of keys (four pages each) that all the rows it serves see together: a
    long row among short ones gets more workgroups, and a recorded step adapts as its requests grow. The
    mixer says through ``uses_query_tiles()`` whether its sizes and dtype take those kernels."""

    RUN_OF_KEYS = ops.DECODE_SPLIT_PAGES * ops.PAGE_SIZE

    def uses_query_tiles(self) -> bool:
        raise NotImplementedError

    def step_arrays_key(self):
        return ("query_tiles", ops.QUERY_TILE, self.RUN_OF_KEYS) if self.uses_query_tiles() else None

    def _decode_work(self, batch) -> int:
        single = batch.num_rows if batch.all_decode else batch.decode_prefix    # the rows that go to the decode kernel
        positions = np.asarray(batch.host_row_pos[:single], dtype=np.int64)
        return int(np.sum((positions + self.RUN_OF_KEYS) // self.RUN_OF_KEYS))

    def step_arrays(self, batch):
        seg_row0 = batch.host_seg_row0
        tile_seg, tile_row0 = ops.query_tiles(seg_row0)
        # Workgroups start in the order of the tiles: those that see the most keys go first, the short
        # ones fill in behind. The tiles of the leading single rows stay in front (they go to the
        # decode kernel and their tiles are skipped).
        if len(tile_seg) - batch.decode_prefix > 1 and not batch.all_decode:
            tile_seg, tile_row0 = np.asarray(tile_seg, dtype=np.int32), np.asarray(tile_row0, dtype=np.int32)
            tile_end = np.minimum(tile_row0 + ops.QUERY_TILE, np.asarray(seg_row0, dtype=np.int32)[tile_seg + 1])
            keys_seen = batch.host_row_pos[tile_end - 1].astype(np.int64)
            keys_seen[:batch.decode_prefix] = np.iinfo(np.int64).max
            order = np.argsort(-keys_seen, kind="stable")
            tile_seg, tile_row0 = tile_seg[order], tile_row0[order]
        return {"tile_seg": np.asarray(tile_seg, dtype=np.int32), "tile_row0": np.asarray(tile_row0, dtype=np.int32),
                "decode_work": np.asarray([self._decode_work(batch)], dtype=np.int32)}

    def refresh_step_arrays(self, batch, arrays) -> None:
        arrays["decode_work"][0] = self._decode_work(batch)     # the tiles of single rows never change


@register_mixer("gqa_attention")
class GQAttention(QueryTileArrays, Mixer):
    graph_safe = True
    accepts_lazy_norm = True
    # Up to this many rows a decode step forms queries and keys inside the attention kernel (at 8 rows
    # 18.9 us against 15.4 + 4.9 us in two kernels); with many rows the attention is bound by reading
    # the cache and the work in front of it only delays every workgroup (64 rows: 74.1 against 65.9 + 7.2 us).
    FUSED_DECODE_ROWS = 16

    def __init__(self, spec):
        super().__init__(spec)
        self.hidden = int(spec["hidden_size"])
        self.num_heads = int(spec["num_heads"])
        self.num_kv_heads = int(spec["num_kv_heads"])
        self.head_dim = int(spec["head_dim"])
        self.v_head_dim = int(spec.get("v_head_dim") or self.head_dim)
        self.qk_norm = bool(spec.get("qk_norm", False))
        self.qk_norm_eps = float(spec.get("qk_norm_eps", 1e-6)) if self.qk_norm else 1.0
        self.window = spec.get("window")
        self.chunk = int(spec.get("chunk") or 0)
        self.softcap = float(spec.get("score_softcap") or 0.0)
        self.keep_first = int(spec.get("keep_first") or 0)
        self.has_sink = bool(spec.get("sink", False))
        self.unit_sink = spec.get("sink") == "unit"
        self.values_are_keys = spec.get("values", "projected") == "keys"
        self.conv_taps = int(spec.get("qk_conv") or 0)
        self.qk_bias = bool(spec.get("qk_bias", False))
        exponent = spec.get("distance_slope_exponent")
        self.slope_exponent = None if exponent is None else float(exponent)
        temperature = spec.get("query_temperature")
        self.q_temperature = None if temperature is None else build_part(
            "position", PartSpec("query_temperature", {"coef": float(temperature[0]), "every": int(temperature[1])}))
        self.shared_kv = bool(spec.get("shared_kv", False))
        self.scale = float(spec.get("softmax_scale", self.head_dim ** -0.5))
        self.bias = bool(spec.get("bias", False))
        self.names = {**_DEFAULT_NAMES, **dict(spec.get("names", {}))}
        # what follows a tensor's name in the checkpoint: ".weight" / ".bias" unless the layout has none
        self.weight_suffix = spec.get("weight_suffix", ".weight")
        self.position = build_part("position", spec["position"])
        if self.num_heads % self.num_kv_heads:
            raise ConfigError(f"{self.num_heads} heads are not a multiple of {self.num_kv_heads} kv heads")
        if max(self.head_dim, self.v_head_dim) > ops.MAX_PLAIN_HEAD_DIM:
            raise ConfigError(f"head_dim {self.head_dim} / value size {self.v_head_dim} exceeds the kernels' limit of {ops.MAX_PLAIN_HEAD_DIM}")
        if self.bias and self.weight_suffix != ".weight":
            raise ConfigError("biases need the '.weight' / '.bias' tensor names")
        if self.window is not None and int(self.window) <= 0:
            raise ConfigError("an attention window must be positive (or None for all keys)")
        if self.chunk < 0 or self.softcap < 0:
            raise ConfigError("an attention chunk and a soft cap on the scores must be positive (or 0 / None for none)")
        if self.keep_first < 0 or (self.keep_first and self.chunk):
            raise ConfigError("first keys are kept beside a window (a non-negative number of them), not beside chunks")
        if self.shared_kv and (self.bias or self.qk_norm):
            raise ConfigError("a layer that reads another layer's keys and values has no biases and no per-head norms here")
        if spec.get("values", "projected") not in ("projected", "keys"):
            raise ConfigError(f"an attention's values are 'projected' or 'keys', not {spec.get('values')!r}")
        if self.values_are_keys and (self.v_head_dim != self.head_dim or self.shared_kv):
            raise ConfigError("values that are the keys have the keys' size, in a layer with keys of its own")
        if (self.conv_taps or self.qk_bias) and (self.shared_kv or self.bias):
            raise ConfigError("convolutions and biases on q and k alone go with a layer's own keys and no other biases")
        if not 0 <= self.conv_taps <= 16:
            raise ConfigError(f"a short convolution of {self.conv_taps} taps (1..16, or 0 for none)")

    @property
    def qk_width(self) -> int:
        return (self.num_heads + self.num_kv_heads) * self.head_dim

    def cache_need(self):
        paged = PagedKV(self.num_kv_heads, self.head_dim, None if self.window is None else int(self.window),
                        None if self.v_head_dim == self.head_dim else self.v_head_dim, self.chunk or None,
                        self.keep_first if self.window is not None else 0)
        if self.conv_taps > 1:      # the convolutions' memory lives in the request's slot beside the pages
            return {"kv": paged, "conv": FixedState((self.qk_width, self.conv_taps - 1), torch.float32)}
        return paged

    def _name(self, which: str, leaf: str = "weight") -> str:
        if leaf == "weight":
            return f"{self.prefix}{self.names[which]}{self.weight_suffix}"
        return f"{self.prefix}{self.names[which]}.{leaf}"

    def tensors(self) -> Dict[str, TensorDecl]:
        q_width, kv_width = self.num_heads * self.head_dim, self.num_kv_heads * self.head_dim
        declared = {
            self._name("q"): TensorDecl((q_width, self.hidden)),
            self._name("k"): TensorDecl((kv_width, self.hidden)),
            self._name("v"): TensorDecl((self.num_kv_heads * self.v_head_dim, self.hidden)),
            self._name("o"): TensorDecl((self.hidden, self.num_heads * self.v_head_dim)),
        }
        if self.shared_kv:
            del declared[self._name("k")], declared[self._name("v")]
        if self.values_are_keys:
            del declared[self._name("v")]
        if self.qk_bias:
            declared[self.prefix + self.names["q_bias"]] = TensorDecl((q_width,), "vector", "bias")
            declared[self.prefix + self.names["k_bias"]] = TensorDecl((kv_width,), "vector", "bias")
        if self.conv_taps:
            declared[self.prefix + self.names["q_conv"]] = TensorDecl((q_width, self.conv_taps), "vector", "conv")
            declared[self.prefix + self.names["k_conv"]] = TensorDecl((kv_width, self.conv_taps), "vector", "conv")
        if self.has_sink and not self.unit_sink:
            declared[self._name("sink")] = TensorDecl((self.num_heads,), "vector", "bias")
        if self.bias:
            declared[self._name("q", "bias")] = TensorDecl((q_width,), "vector", "bias")
            declared[self._name("k", "bias")] = TensorDecl((kv_width,), "vector", "bias")
            declared[self._name("v", "bias")] = TensorDecl((kv_width,), "vector", "bias")
            declared[self._name("o", "bias")] = TensorDecl((self.hidden,), "vector", "bias")
        if self.qk_norm:
            declared[self._name("q_norm")] = TensorDecl((self.head_dim,), "vector", "norm")
            declared[self._name("k_norm")] = TensorDecl((self.head_dim,), "vector", "norm")
        return declared

    def bind(self, tensors, dtype, device) -> None:
        super().bind(tensors, dtype, device)
        self.position.bind(tensors, dtype, device)
        self.sinks = tensors[self._name("sink")] if self.has_sink and not self.unit_sink else None
        if self.unit_sink:
            self.sinks = torch.zeros((self.num_heads,), dtype=torch.float32, device=device)
        self.slopes = None
        if self.slope_exponent is not None:
            heads = torch.arange(1, self.num_heads + 1, dtype=torch.float64)
            self.slopes = torch.pow(2.0, -self.slope_exponent * heads / self.num_heads).to(dtype=torch.float32, device=device)
        if self.q_temperature is not None:
            self.q_temperature.bind(tensors, dtype, device)
        self.conv = None
        if self.values_are_keys:
            # queries and keys alone; the values are the keys a second time, written behind them by the convolution
            # (one of a single tap of 1 where the layer has none of its own)
            q, k = tensors[self._name("q")], tensors[self._name("k")]
            if q.dtype != k.dtype:
                raise ConfigError(f"{self.prefix}: q and k projections are stored in different precisions")
            bias = torch.cat([tensors[self.prefix + self.names[n]] for n in ("q_bias", "k_bias")]) if self.qk_bias else None
            self.qkv = Linear(torch.cat([q, k], dim=0), bias)
        elif self.shared_kv:
            self.qkv = Linear(tensors[self._name("q")])        # the queries alone
        else:
            q, k, v = (tensors[self._name(n)] for n in ("q", "k", "v"))
            if not (q.dtype == k.dtype == v.dtype):
                raise ConfigError(f"{self.prefix}: q, k and v projections are stored in different precisions")
            # one operand for the three projections: rows are q heads, then k heads, then v heads
            bias = torch.cat([tensors[self._name(n, "bias")] for n in ("q", "k", "v")]) if self.bias else None
            if self.qk_bias:
                bias = torch.cat([tensors[self.prefix + self.names["q_bias"]], tensors[self.prefix + self.names["k_bias"]],
                                  torch.zeros((v.shape[0],), dtype=torch.float32, device=device)])
            self.qkv = Linear(torch.cat([q, k, v], dim=0), bias)
        if self.conv_taps:
            self.conv = torch.cat([tensors[self.prefix + self.names[n]] for n in ("q_conv", "k_conv")], dim=0).contiguous()
        elif self.values_are_keys:
            self.conv = torch.ones((self.qk_width, 1), dtype=torch.float32, device=device)
        self._no_conv_state = None
        self.out = Linear(tensors[self._name("o")], tensors[self._name("o", "bias")] if self.bias else None)
        self.q_norm_weight = tensors[self._name("q_norm")] if self.qk_norm else None
        self.k_norm_weight = tensors[self._name("k_norm")] if self.qk_norm else None

    def uses_query_tiles(self) -> bool:
        return getattr(self, "dtype", None) == torch.bfloat16 and ops.attention_is_tiled(self.head_dim) \
            and ops.attention_is_tiled(self.v_head_dim)

    def attend(self, h, ctx, cache) -> torch.Tensor:
        """The heads' outputs [rows, heads * v_head_dim] in the activation dtype, the step's keys and
        values appended to the cache on the way."""
        qkv = self.qkv.forward(h, out_dtype=torch.float32)      # normed, rotated and rounded once, below
        if isinstance(cache, dict):
            memory, cache = cache.get("conv"), cache["kv"]
        else:
            memory = None
        if self.conv is not None:
            # q and k pass their convolutions (their memory in the request's slot moves on); where the values are the
            # keys, the keys leave twice: [q | k | k], the second time as the values, which no norm touches
            if memory is not None:
                state = memory.state
            else:
                slots = int(ctx.seg_slot.numel()) + 1
                if self._no_conv_state is None:
                    self._no_conv_state = torch.zeros((1 << 16, self.qk_width, 0), dtype=torch.float32, device=self.device)
                state = self._no_conv_state
            echo = (self.num_heads * self.head_dim, self.num_kv_heads * self.head_dim) if self.values_are_keys else None
            moved = ops.causal_conv(qkv[:, :self.qk_width], self.conv, None, state, ctx.row_seg, ctx.seg_row0, ctx.seg_slot,
                                    ctx.num_segments, single_rows=ctx.all_decode, echo=echo)
            if self.values_are_keys:
                qkv = moved
            else:
                qkv[:, :self.qk_width] = moved
        q_factor = ctx.position_tables(self.q_temperature) if self.q_temperature is not None else None
        cos, sin = ctx.position_tables(self.position)
        interleaved = bool(getattr(self.position, "interleaved", False))
        own = ctx.step_arrays(self) if self.step_arrays_key() is not None else {}
        if self.shared_kv and cache.writes:
            raise ConfigError(f"{self.prefix}: the layer has no keys and values of its own; its schedule entry must read another's cache entry")
        mask = {"keep_first": self.keep_first if self.window else 0, "sinks": self.sinks, "slopes": self.slopes}
        if ctx.all_decode and ctx.num_rows <= self.FUSED_DECODE_ROWS and qkv.dtype == torch.float32 and self.step_arrays_key() is not None:
            # a few single-token segments on the matrix cores: norm, rotation, cache write and attention in one kernel
            return ops.attention_decode_fused(
                qkv, self.num_heads, self.num_kv_heads, self.head_dim, self.q_norm_weight, self.k_norm_weight, self.qk_norm_eps,
                cos, sin, self.position.rotary_dim, cache.k_pages, cache.v_pages, cache.block_table, ctx.row_seg, ctx.row_pos,
                self.scale, ctx.max_context, int(self.window or 0), write_kv=cache.writes,
                decode_work=own.get("decode_work"), v_dim=self.v_head_dim, chunk=self.chunk, softcap=self.softcap,
                interleaved=interleaved, q_only=self.shared_kv, q_row_scale=q_factor, **mask)
        q = ops.qk_norm_rope_kv_write(
            qkv, self.num_heads, self.num_kv_heads, self.head_dim, self.q_norm_weight, self.k_norm_weight,
            self.qk_norm_eps, cos, sin, self.position.rotary_dim, cache.k_pages, cache.v_pages, cache.block_table,
            ctx.row_seg, ctx.row_pos, write_kv=cache.writes, v_dim=self.v_head_dim, interleaved=interleaved, q_only=self.shared_kv,
            q_row_scale=q_factor)
        return ops.attention(q, self.num_heads, self.num_kv_heads, self.head_dim, cache.k_pages, cache.v_pages,
                             cache.block_table, ctx, self.scale, int(self.window or 0),
                             tile_seg=own.get("tile_seg"), tile_row0=own.get("tile_row0"), decode_work=own.get("decode_work"),
                             v_dim=self.v_head_dim, chunk=self.chunk, softcap=self.softcap, **mask)

    def forward(self, h, residual, ctx, cache):
        return self.out.accumulate(self.attend(h, ctx, cache), residual, then=getattr(ctx, "upcoming_norm", None))

    def output(self, h, ctx, cache) -> torch.Tensor:
        """The mixer's output as float32 rows of its own (for arrangements that do something to it
        before it joins the residual stream)."""
        return self.out.forward(self.attend(h, ctx, cache), out_dtype=torch.float32)
