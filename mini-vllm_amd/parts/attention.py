"""Softmax attention over the paged cache, with grouped key/value heads.

Reference: minivllm/models/models/qwen3.py:26-101 (projection, per-head q/k norm before the
rotary embedding, output projection) and minivllm/models/layers/attention.py:46-92 (cache
write, then causal attention over the request's keys). ``scale`` is head_dim^-0.5
(qwen3.py:32). ``window`` is the number of tokens to the left of a query that it sees besides
itself (attention.py:56-60); None sees all.

Every size is a parameter of the spec. q, k and v are packed into one matrix product; the
per-head norms, the rotary embedding and the cache write are one kernel.

Beyond the reference's layer the spec has, each off by default: values of another size than keys
(``value_dim``); ``chunk``: a query sees only the keys of its own chunk of the sequence (positions
with equal ``position // chunk``, counted from the sequence's start); ``weighting = "sigmoid"``: the
weight of a visible key is sigmoid(score * scale + score_bias[head]) and the weights are not
normalised over the keys; ``head_gate``: head h's output is multiplied by sigmoid(W_gate x)[h], one
number per head, read from the same packed product as q, k and v; ``keep_first`` (with a window): a
query also sees the sequence's first ``keep_first`` positions however far back they lie, at their true
positions; ``value_from_key``: there is no value projection, the values are the keys as projected,
before norm and rotation. Softmax weighting with any of the last three runs ``_forward_kept``.

``unit_norm_after_rotation``: q and k are rotated first and then divided by their root mean square per head
(x / sqrt(mean(x^2) + qk_norm_eps), no weight). ``value_mix``: values are shared between layers of a model
within a token: a layer with ``value_mix = "source"`` leaves the values it projected for the step's tokens in
``ctx.carry[value_mix_key]``; a layer with ``"blend"`` caches (1 - m) v + m v_source instead of its own v,
with m its stored number ``value_mix`` (both must have the same kv heads and value size). Softmax weighting
with either of these, or with values of another size than keys, runs ``_forward_rotated``.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Optional, Tuple

import torch

from .base import (CacheNeed, KeepAll, KeepChunks, KeepWindow, KeepWindowAndFirst, KeyValueNeed, Mixer, PartSpec, Runtime,
                   TensorDecl, register_mixer)


@dataclass(frozen=True)
class AttentionSpec(PartSpec):
    kind = "attention"
    hidden_size: int = 0
    num_heads: int = 0
    num_kv_heads: int = 0
    head_dim: int = 0
    scale: float = 1.0
    qk_norm: bool = False
    qk_norm_eps: float = 1e-6
    bias: bool = False
    window: Optional[int] = None
    position: Optional[PartSpec] = None
    shares_kv: bool = False        # no k/v of its own: reads the cache of the call named by the plan
    value_dim: Optional[int] = None          # None: head_dim
    weighting: str = "softmax"               # or "sigmoid"
    score_bias: bool = False                 # a learned number per head added to the scaled score (sigmoid weighting)
    chunk: Optional[int] = None
    head_gate: bool = False
    # chunk sizes of every call that reads this call's cache, its own among them (they decide how long
    # pages stay); empty: its own ``chunk`` alone. ``cache_keeps_all``: some reader sees all keys.
    cache_chunks: Tuple[int, ...] = ()
    cache_keeps_all: bool = False
    keep_first: int = 0                      # with a window: the sequence's first positions stay visible
    value_from_key: bool = False             # values = keys as projected (no value projection)
    unit_norm_after_rotation: bool = False   # q, k <- x / rms(x) per head, behind the rotation, without a weight
    value_mix: Optional[str] = None          # "source" or "blend", see above
    value_mix_key: str = ""

    @property
    def q_dim(self) -> int:
        return self.num_heads * self.head_dim

    @property
    def kv_dim(self) -> int:
        return self.num_kv_heads * self.head_dim

    @property
    def v_head_dim(self) -> int:
        return self.head_dim if self.value_dim is None else self.value_dim

    @property
    def v_dim(self) -> int:
        return self.num_kv_heads * self.v_head_dim

    @property
    def out_dim(self) -> int:
        return self.num_heads * self.v_head_dim

    @property
    def plain(self) -> bool:
        """The reference's layer: softmax over all keys or a window, values as large as keys."""
        return (self.weighting == "softmax" and self.chunk is None and self.value_dim in (None, self.head_dim)
                and not self.head_gate and not self.score_bias and not self.keep_first and not self.value_from_key
                and not self.unit_norm_after_rotation and self.value_mix is None)

    @property
    def rotated(self) -> bool:
        """Softmax with the unit norm behind the rotation, values shared between layers, or values of a size of their own."""
        return (self.weighting == "softmax" and self.chunk is None and not self.score_bias and not self.bias
                and not self.qk_norm and not self.head_gate and not self.keep_first and not self.value_from_key
                and not self.shares_kv
                and (self.unit_norm_after_rotation or self.value_mix is not None or self.value_dim not in (None, self.head_dim)))

    @property
    def kept(self) -> bool:
        """Softmax over a window (or all keys) with kept first positions, head gates or values taken from the keys."""
        return (self.weighting == "softmax" and self.chunk is None and self.value_dim in (None, self.head_dim)
                and not self.score_bias and not self.bias and not self.qk_norm and not self.plain and not self.rotated
                and not self.unit_norm_after_rotation and self.value_mix is None)


@register_mixer(AttentionSpec.kind)
class Attention(Mixer):
    spec_class = AttentionSpec
    accepts_pending_norm = True      # the input is used by one packed product only
    accepts_fold = True              # the output comes from one product

    @classmethod
    def tensors(cls, spec: AttentionSpec) -> Dict[str, TensorDecl]:
        t = {"q": TensorDecl((spec.q_dim, spec.hidden_size)), "o": TensorDecl((spec.hidden_size, spec.out_dim))}
        if not spec.shares_kv:
            t["k"] = TensorDecl((spec.kv_dim, spec.hidden_size))
            if not spec.value_from_key:
                t["v"] = TensorDecl((spec.v_dim, spec.hidden_size))
        if spec.score_bias:
            t["score_bias"] = TensorDecl((spec.num_heads,), init="zeros_normal")
        if spec.head_gate:
            t["head_gate"] = TensorDecl((spec.num_heads, spec.hidden_size))
        if spec.value_mix == "blend":
            t["value_mix"] = TensorDecl((), init="zeros_normal")
        if spec.bias:
            t["q_bias"] = TensorDecl((spec.q_dim,), init="zeros_normal")
            t["o_bias"] = TensorDecl((spec.hidden_size,), init="zeros_normal")
            if not spec.shares_kv:
                t["k_bias"] = TensorDecl((spec.kv_dim,), init="zeros_normal")
                t["v_bias"] = TensorDecl((spec.kv_dim,), init="zeros_normal")
        if spec.qk_norm:
            t["q_norm"] = TensorDecl((spec.head_dim,), init="ones_normal")
            if not spec.shares_kv:
                t["k_norm"] = TensorDecl((spec.head_dim,), init="ones_normal")
        return t

    @classmethod
    def cache_need(cls, spec: AttentionSpec) -> Optional[CacheNeed]:
        if spec.shares_kv:
            return None
        if spec.chunk is not None or spec.cache_chunks:
            sizes = tuple(sorted(set(spec.cache_chunks or (spec.chunk,))))
            retention = KeepAll() if spec.cache_keeps_all else KeepChunks(sizes)
        else:
            if spec.window is None or spec.cache_keeps_all:
                retention = KeepAll()
            elif spec.keep_first > 0:
                retention = KeepWindowAndFirst(spec.window, spec.keep_first)
            else:
                retention = KeepWindow(spec.window)
        return KeyValueNeed(retention=retention, num_kv_heads=spec.num_kv_heads, head_dim=spec.head_dim,
                            value_dim=spec.value_dim)

    def __init__(self, spec: AttentionSpec, tensors: Dict[str, torch.Tensor], rt: Runtime,
                 position: Optional[object] = None):
        if spec.num_heads % spec.num_kv_heads:
            raise ValueError(f"{spec.num_heads} query heads are not a multiple of {spec.num_kv_heads} kv heads")
        if spec.weighting not in ("softmax", "sigmoid"):
            raise ValueError(f"attention weighting must be 'softmax' or 'sigmoid', got {spec.weighting!r}")
        if spec.value_mix not in (None, "source", "blend") or (spec.value_mix and not spec.value_mix_key):
            raise ValueError(f"value_mix must be None, 'source' or 'blend' with a key, got {spec.value_mix!r}, {spec.value_mix_key!r}")
        if (spec.unit_norm_after_rotation or spec.value_mix) and not spec.rotated:
            raise NotImplementedError("the unit norm behind the rotation and values shared between layers are built for softmax "
                                      "weighting over all keys or a window, without biases, weighted q/k norms, gates or a shared cache")
        if not spec.plain and not spec.kept and not spec.rotated and (spec.weighting != "sigmoid" or spec.bias):
            raise NotImplementedError("chunks, a value size of its own and a score bias are built for sigmoid weighting "
                                      "without projection biases; kept first positions, head gates and values taken from "
                                      "the keys also for softmax weighting without biases and query/key norms")
        if spec.keep_first < 0 or (spec.value_from_key and (spec.shares_kv or spec.v_head_dim != spec.head_dim)):
            raise ValueError("values taken from the keys have the keys' size and a cache of their own; keep_first is >= 0")
        if (spec.keep_first or spec.value_from_key) and not spec.kept:
            raise NotImplementedError("kept first positions and values taken from the keys are built for softmax weighting")
        self.spec = spec
        self.rt = rt
        parts = ["q"] if spec.shares_kv else (["q", "k"] if spec.value_from_key else ["q", "k", "v"])
        if spec.head_gate:
            parts = parts + ["head_gate"]
        dtypes = {tensors[p].dtype for p in parts}
        if len(dtypes) != 1:
            raise ValueError(f"q, k and v projections are stored in different dtypes {dtypes}; cannot pack them")
        self.w_qkv = tensors["q"] if len(parts) == 1 else torch.cat([tensors[p] for p in parts], dim=0).contiguous()
        self.b_qkv = None
        self.b_o = None
        if spec.bias:
            self.b_qkv = tensors["q_bias"] if len(parts) == 1 else torch.cat(
                [tensors[p + "_bias"] for p in parts], dim=0).contiguous()
            self.b_o = tensors["o_bias"]
        self.w_o = tensors["o"]
        self.q_norm = tensors.get("q_norm")
        self.k_norm = tensors.get("k_norm")
        self.value_mix = tensors.get("value_mix")
        self.position = position
        self.rotary = position.rotary() if position is not None else None
        if position is not None and self.rotary is None and not hasattr(position, "apply"):
            raise ValueError("a position encoding must offer rotary() or apply()")
        self.width = spec.q_dim + (0 if spec.shares_kv else spec.kv_dim + (0 if spec.value_from_key else spec.v_dim))
        self.gate_off = self.width                        # the head gates come last in the packed rows
        if spec.head_gate:
            self.width += spec.num_heads
        self.score_bias = tensors.get("score_bias")
        if self.score_bias is not None:
            self.score_bias = self.score_bias.to(torch.float32)
        if self.w_qkv.shape[0] != self.width:
            raise ValueError(f"the packed projection has {self.w_qkv.shape[0]} rows, expected {self.width}")
        if not spec.plain and self.width % 8:
            # rows of the packed product keep a pitch of a multiple of 8 elements (zero rows at the end)
            pad = (-self.width) % 8
            self.w_qkv = torch.cat([self.w_qkv, torch.zeros((pad, spec.hidden_size), dtype=self.w_qkv.dtype,
                                                            device=self.w_qkv.device)], dim=0).contiguous()
            self.width += pad

    def first_product(self):
        return self.w_qkv.shape[0], self.w_qkv.shape[1], False

    def forward(self, x: torch.Tensor, ctx, call: int, fold=None) -> torch.Tensor:
        spec, rt, ops = self.spec, self.rt, self.rt.ops
        if spec.rotated:
            return self._forward_rotated(x, ctx, call)
        if spec.kept:
            return self._forward_kept(x, ctx, call)
        if not spec.plain:
            return self._forward_sigmoid(x, ctx, call)
        n = x.shape[0]
        ws = rt.workspace
        qkv = ws.get("attn.qkv", (n, self.width), rt.dtype)
        ops.gemm(x, self.w_qkv, qkv, self.b_qkv)
        kv = ctx.kv(call)
        table, interleaved = (self.rotary if self.rotary is not None else (None, False))
        if self.position is not None and self.rotary is None:
            q3 = qkv[:, :spec.q_dim].unflatten(1, (spec.num_heads, spec.head_dim))
            k3 = None if spec.shares_kv else qkv[:, spec.q_dim:spec.q_dim + spec.kv_dim].unflatten(
                1, (spec.num_kv_heads, spec.head_dim))
            if spec.qk_norm:
                raise NotImplementedError("a position encoding without a rotary table cannot follow the fused "
                                          "q/k norm; give it a table or leave qk_norm off")
            self.position.apply(q3, k3, ctx)
        attn = ws.get("attn.out", (n, spec.q_dim), rt.dtype)
        plan = ctx.attention_plan
        if plan is not None and plan.decode_only:
            # a decode step: norm, rotation, cache write and attention in one kernel where it is taken
            if ops.attention_decode_fused(qkv, attn, kv.k_pages, kv.v_pages, kv.block_table, kv.page_size,
                                          ctx.positions, ctx.token_seq, spec.num_heads, spec.num_kv_heads,
                                          spec.head_dim, spec.scale, spec.window, plan, self.q_norm, self.k_norm,
                                          spec.qk_norm_eps, table, interleaved, not spec.shares_kv,
                                          rope_rows=ctx.position_rows.get(self.position)):
                y = ws.get("mixer.out", (n, spec.hidden_size), rt.dtype)
                return ops.gemm(attn, self.w_o, y, self.b_o, defer_sum=True, fold=fold) or y
        ops.qk_norm_rope_store(
            qkv, spec.num_heads, spec.num_kv_heads, spec.head_dim, ctx.positions, ctx.token_seq,
            self.q_norm, self.k_norm, spec.qk_norm_eps, table, interleaved,
            None if spec.shares_kv else kv.k_pages, None if spec.shares_kv else kv.v_pages,
            None if spec.shares_kv else kv.block_table, kv.page_size)
        ops.attention(qkv[:, :spec.q_dim] if self.width != spec.q_dim else qkv, attn, kv.k_pages, kv.v_pages,
                      kv.block_table, kv.page_size, ctx.positions, ctx.token_seq, spec.num_heads,
                      spec.num_kv_heads, spec.head_dim, spec.scale, spec.window, plan=ctx.attention_plan)
        y = ws.get("mixer.out", (n, spec.hidden_size), rt.dtype)
        # (the sums of a product whose K was split may be left to the next norm)
        return ops.gemm(attn, self.w_o, y, self.b_o, defer_sum=True, fold=fold) or y

    def _forward_sigmoid(self, x: torch.Tensor, ctx, call: int) -> torch.Tensor:
        """Sigmoid weighting (chunks, a window or all keys; values of any size; score bias; head gates)."""
        spec, rt, ops, ws = self.spec, self.rt, self.rt.ops, self.rt.workspace
        n = x.shape[0]
        packed = ws.get("attn.qkv", (n, self.width), rt.dtype)
        ops.gemm(x, self.w_qkv, packed)
        kv = ctx.kv(call)
        table, interleaved = (self.rotary if self.rotary is not None else (None, False))
        if self.position is not None and self.rotary is None:
            raise NotImplementedError("sigmoid attention takes its rotation from a rotary table")
        own = not spec.shares_kv
        ops.qk_norm_rope_store(
            packed, spec.num_heads, spec.num_kv_heads, spec.head_dim, ctx.positions, ctx.token_seq,
            self.q_norm, self.k_norm, spec.qk_norm_eps, table, interleaved,
            kv.k_pages if own else None, kv.v_pages if own else None, kv.block_table if own else None, kv.page_size,
            value_dim=spec.v_head_dim)
        attn = ws.get("attn.out", (n, spec.out_dim), rt.dtype)
        gate = packed[:, self.gate_off:self.gate_off + spec.num_heads] if spec.head_gate else None
        ops.attention_sigmoid(packed[:, :spec.q_dim], attn, kv.k_pages, kv.v_pages, kv.block_table, kv.page_size,
                              ctx.positions, ctx.token_seq, spec.num_heads, spec.num_kv_heads, spec.head_dim,
                              spec.v_head_dim, spec.scale, spec.chunk, spec.window, self.score_bias, gate,
                              plan=ctx.attention_plan)
        y = ws.get("mixer.out", (n, spec.hidden_size), rt.dtype)
        return ops.gemm(attn, self.w_o, y, self.b_o, defer_sum=True) or y

    def _forward_kept(self, x: torch.Tensor, ctx, call: int) -> torch.Tensor:
        """Softmax weighting over a window with kept first positions, head gates, values taken from the keys."""
        spec, rt, ops, ws = self.spec, self.rt, self.rt.ops, self.rt.workspace
        if not isinstance(x, torch.Tensor):
            x = x.materialize()
        n = x.shape[0]
        packed = ws.get("attn.qkv", (n, self.width), rt.dtype)
        ops.gemm(x, self.w_qkv, packed)
        kv = ctx.kv(call)
        table, interleaved = (self.rotary if self.rotary is not None else (None, False))
        if self.position is not None and self.rotary is None:
            raise NotImplementedError("this attention takes its rotation from a rotary table")
        own = not spec.shares_kv
        held = spec.q_dim + (0 if not own else spec.kv_dim + (0 if spec.value_from_key else spec.v_dim))
        ops.qk_norm_rope_store(
            packed, spec.num_heads, spec.num_kv_heads, spec.head_dim, ctx.positions, ctx.token_seq,
            None, None, spec.qk_norm_eps, table, interleaved,
            kv.k_pages if own else None, kv.v_pages if own else None, kv.block_table if own else None, kv.page_size,
            value_from_key=spec.value_from_key, extra_columns=self.width - held)
        attn = ws.get("attn.out", (n, spec.out_dim), rt.dtype)
        gate = packed[:, self.gate_off:self.gate_off + spec.num_heads] if spec.head_gate else None
        ops.attention(packed[:, :spec.q_dim], attn, kv.k_pages, kv.v_pages, kv.block_table, kv.page_size, ctx.positions,
                      ctx.token_seq, spec.num_heads, spec.num_kv_heads, spec.head_dim, spec.scale, spec.window,
                      plan=ctx.attention_plan, keep_first=spec.keep_first, gate=gate)
        y = ws.get("mixer.out", (n, spec.hidden_size), rt.dtype)
        return ops.gemm(attn, self.w_o, y, defer_sum=True) or y

    def _forward_rotated(self, x: torch.Tensor, ctx, call: int) -> torch.Tensor:
        """Softmax weighting with the unit norm behind the rotation, values blended with another layer's, values of any size."""
        spec, rt, ops, ws = self.spec, self.rt, self.rt.ops, self.rt.workspace
        if not isinstance(x, torch.Tensor):
            x = x.materialize()
        n = x.shape[0]
        # the layer whose values the later ones blend in keeps its rows in a buffer of its own for the rest of the step
        name = f"attn.qkv.{spec.value_mix_key}" if spec.value_mix == "source" else "attn.qkv"
        packed = ws.get(name, (n, self.width), rt.dtype)
        ops.gemm(x, self.w_qkv, packed)
        kv = ctx.kv(call)
        table, interleaved = (self.rotary if self.rotary is not None else (None, False))
        if self.position is not None and self.rotary is None:
            raise NotImplementedError("this attention takes its rotation from a rotary table")
        v_off = spec.q_dim + spec.kv_dim
        mix_rows = None
        if spec.value_mix == "source":
            ctx.carry[spec.value_mix_key] = packed[:, v_off:v_off + spec.v_dim]
        elif spec.value_mix == "blend":
            mix_rows = ctx.carry.get(spec.value_mix_key)
            if mix_rows is None or mix_rows.shape[0] != n or mix_rows.shape[1] != spec.v_dim:
                raise RuntimeError(f"no layer in front of this one left values of {spec.v_dim} columns under {spec.value_mix_key!r}")
        ops.qkv_rotate_norm_store(packed, spec.num_heads, spec.num_kv_heads, spec.head_dim, spec.v_head_dim, ctx.positions,
                                  ctx.token_seq, table, interleaved, spec.unit_norm_after_rotation, spec.qk_norm_eps,
                                  kv.k_pages, kv.v_pages, kv.block_table, kv.page_size, mix_rows=mix_rows,
                                  mix_weight=self.value_mix if mix_rows is not None else None)
        attn = ws.get("attn.out", (n, spec.out_dim), rt.dtype)
        ops.attention(packed[:, :spec.q_dim], attn, kv.k_pages, kv.v_pages, kv.block_table, kv.page_size, ctx.positions,
                      ctx.token_seq, spec.num_heads, spec.num_kv_heads, spec.head_dim, spec.scale, spec.window,
                      plan=ctx.attention_plan, value_dim=spec.v_head_dim)
        y = ws.get("mixer.out", (n, spec.hidden_size), rt.dtype)
        return ops.gemm(attn, self.w_o, y, defer_sum=True) or y
