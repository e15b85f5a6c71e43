"""Softmax attention whose keys and values are linear maps of one cached latent per token.

From the mixer's input h:

    c_q = rmsnorm(W_dq h) * w_q_norm,   q = W_uq c_q                  (heads x [plain_dim | rot_dim])
    W_dkv h = [down (kv_rank) | key part (rot_dim)]
    c   = rmsnorm(down) * w_kv_norm                                    (the latent)
    k_rot = rot(key part, position)                                    (one for all heads)

Head h's key is [W_uk,h c | k_rot] and its value W_uv,h c; the score of query i and key j <= i is
(q_plain . W_uk c_j + rot(q_rot) . k_rot,j) * scale, softmax over the visible keys. The heads'
outputs are concatenated, multiplied by sigmoid(W_g h) when ``output_gate`` is set (with ``head_gate`` W_g has
one row a head and the whole head is multiplied by that one number), and projected by W_o.

``rot_neighbours``: the rotation pairs channel 2i with 2i + 1 instead of i with i + rot_dim / 2. A score only sums
products of a query's channel with the same channel of a key, so it does not change when the rotated channels of
both are put in another order: the rows of W_uq and W_dkv that make them are reordered once, when the part is built
(even channels first, then the odd ones), and the kernels rotate in half-split pairs as before.

Only [c | k_rot] is cached, one row of ``kv_rank + rot_dim`` numbers per token, and c once more in
the slot-contiguous layout that the MFMA kernel's second product reads (``LatentNeed``). Keys and values are never expanded: the query is carried into the latent's space
(W_uk,h^T q_plain), attention runs on the cached rows with the latent as the value, and W_uv,h is
applied to the weighted sum of latents. Norms, rotation, scores, weights and sums are float32.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Optional, Tuple

import torch

from .base import CacheNeed, KeepAll, Mixer, PartSpec, Retention, Runtime, TensorDecl, register_mixer


@dataclass(frozen=True)
class LatentNeed(CacheNeed):
    """One row per token: the latent and the rotated key part side by side (``latent``). With ``latent_dim`` the latent
    is kept once more with a page's slots side by side (``latent_t`` [latent_dim, slot]): the second product of an MFMA
    attention kernel reads eight neighbouring keys of one channel in one load from there."""
    retention: Retention
    width: int
    latent_dim: int = 0

    def page_shapes(self, page_size: int) -> Dict[str, Tuple[int, ...]]:
        shapes = {"latent": (page_size, self.width)}
        if self.latent_dim:
            shapes["latent_t"] = (self.latent_dim, page_size)
        return shapes


@dataclass(frozen=True)
class LatentAttentionSpec(PartSpec):
    kind = "latent_attention"
    hidden_size: int = 0
    num_heads: int = 0
    plain_dim: int = 0                  # query/key channels of a head that are not rotated
    rot_dim: int = 0                    # rotated channels: of each query head, and of the one shared key part
    value_dim: int = 0
    q_rank: int = 0
    kv_rank: int = 0
    scale: float = 1.0
    norm_eps: float = 1e-6              # of the two latent norms
    output_gate: bool = False
    head_gate: bool = False             # with output_gate: one gate a head instead of one a channel
    rot_neighbours: bool = False        # the rotation pairs neighbouring channels
    position: Optional[PartSpec] = None     # a rotary encoding over rot_dim channels (None: rot_dim must be 0)


@register_mixer(LatentAttentionSpec.kind)
class LatentAttention(Mixer):
    spec_class = LatentAttentionSpec

    @classmethod
    def tensors(cls, spec: LatentAttentionSpec) -> Dict[str, TensorDecl]:
        hid, H = spec.hidden_size, spec.num_heads
        t = {"dq": TensorDecl((spec.q_rank, hid)), "dq_norm": TensorDecl((spec.q_rank,), init="ones_normal"),
             "uq": TensorDecl((H * (spec.plain_dim + spec.rot_dim), spec.q_rank)),
             "dkv": TensorDecl((spec.kv_rank + spec.rot_dim, hid)), "dkv_norm": TensorDecl((spec.kv_rank,), init="ones_normal"),
             "uk": TensorDecl((H * spec.plain_dim, spec.kv_rank)), "uv": TensorDecl((H * spec.value_dim, spec.kv_rank)),
             "o": TensorDecl((hid, H * spec.value_dim))}
        if spec.output_gate:
            t["g"] = TensorDecl((H if spec.head_gate else H * spec.value_dim, hid))
        return t

    @classmethod
    def cache_need(cls, spec: LatentAttentionSpec) -> Optional[CacheNeed]:
        return LatentNeed(retention=KeepAll(), width=spec.kv_rank + spec.rot_dim, latent_dim=spec.kv_rank)

    def __init__(self, spec: LatentAttentionSpec, tensors: Dict[str, torch.Tensor], rt: Runtime, position: Optional[object] = None):
        if min(spec.num_heads, spec.plain_dim, spec.value_dim, spec.q_rank, spec.kv_rank) < 1 or spec.rot_dim < 0 or spec.rot_dim % 2:
            raise ValueError(f"latent attention: bad sizes {spec}")
        self.spec, self.rt = spec, rt
        self.table = None
        if spec.rot_dim:
            rotary = position.rotary() if position is not None else None
            if rotary is None or rotary[1] or rotary[0].shape[1] != spec.rot_dim:
                raise ValueError("latent attention rotates its rot_dim channels in half-split pairs: it needs a rotary "
                                 "encoding over exactly rot_dim channels")
            self.table = rotary[0]
        if spec.head_gate and not spec.output_gate:
            raise ValueError("latent attention: head_gate says how the output gate is shaped; it needs output_gate")
        names = ["dq", "dkv"] + (["g"] if spec.output_gate else [])
        dtypes = {tensors[p].dtype for p in names}
        if len(dtypes) != 1:
            raise ValueError(f"latent attention: the projections are stored in different dtypes {dtypes}; cannot pack them")
        tensors = dict(tensors)
        if spec.rot_neighbours and spec.rot_dim:
            # rotated channels in the order even, odd: pair (2i, 2i + 1) becomes (i, i + rot_dim / 2)
            dr, dh = spec.rot_dim, spec.plain_dim + spec.rot_dim
            order = torch.cat([torch.arange(0, dr, 2), torch.arange(1, dr, 2)]).to(tensors["dkv"].device)
            rows = torch.cat([torch.arange(spec.kv_rank, device=order.device), spec.kv_rank + order])
            tensors["dkv"] = tensors["dkv"].index_select(0, rows).contiguous()
            head = torch.cat([torch.arange(spec.plain_dim, device=order.device), spec.plain_dim + order])
            rows = (torch.arange(spec.num_heads, device=order.device)[:, None] * dh + head[None, :]).reshape(-1)
            tensors["uq"] = tensors["uq"].index_select(0, rows).contiguous()
        blocks = [tensors[p] for p in names]
        self.gate_offset = spec.q_rank + spec.kv_rank + spec.rot_dim
        pad = (-sum(b.shape[0] for b in blocks)) % 8
        if pad:
            blocks.append(torch.zeros((pad, spec.hidden_size), dtype=blocks[0].dtype, device=blocks[0].device))
        self.w_packed = torch.cat(blocks, dim=0).contiguous()
        self.width = self.w_packed.shape[0]
        self.q_norm = tensors["dq_norm"]
        self.kv_norm = tensors["dkv_norm"].to(self.q_norm.dtype)
        self.w_uq = tensors["uq"]
        # [heads, inputs, outputs]: the stored W_uk is that already; W_uv is stored [heads * value_dim, kv_rank]
        self.w_uk = tensors["uk"].view(spec.num_heads, spec.plain_dim, spec.kv_rank).contiguous()
        self.w_uv = tensors["uv"].view(spec.num_heads, spec.value_dim, spec.kv_rank).transpose(1, 2).contiguous()
        # ... and both as [heads, outputs, inputs], which the MFMA kernel of steps with many rows reads
        self.w_uk_rows = self.w_uk.transpose(1, 2).contiguous()
        self.w_uv_rows = tensors["uv"].view(spec.num_heads, spec.value_dim, spec.kv_rank).contiguous()
        self.w_o = tensors["o"]

    def forward(self, x: torch.Tensor, ctx, call: int) -> torch.Tensor:
        spec, rt, ops, ws = self.spec, self.rt, self.rt.ops, self.rt.workspace
        n, H, R, dr = x.shape[0], spec.num_heads, spec.kv_rank, spec.rot_dim
        packed = ws.get("latent.packed", (n, self.width), rt.dtype)
        ops.gemm(x, self.w_packed, packed)
        kv = ctx.kv(call)
        pages, pages_t = kv.pages["latent"], kv.pages.get("latent_t")
        cq = ws.get("latent.cq", (n, spec.q_rank), rt.dtype)
        ops.latent_prepare(packed, spec.q_rank, R, dr, self.q_norm, self.kv_norm, spec.norm_eps, self.table, ctx.positions,
                           ctx.token_seq, kv.block_table, kv.page_size, cq, pages, pages_t)
        q = ws.get("latent.q", (n, H * (spec.plain_dim + dr)), rt.dtype)
        ops.gemm(cq, self.w_uq, q)
        qa = ws.get("latent.qa", (n, H, R + dr), torch.float32)
        ops.head_linear(q.view(n, H, spec.plain_dim + dr), self.w_uk, qa, ctx.token_seq, tail=dr, table=self.table,
                        positions=ctx.positions, w_rows=self.w_uk_rows)
        mixed = ws.get("latent.mixed", (n, H, R), torch.float32)
        ops.attention_latent(qa, mixed, pages, kv.block_table, kv.page_size, ctx.positions, ctx.token_seq, H, R, dr,
                             spec.scale, plan=ctx.attention_plan, pages_t=pages_t)
        heads = ws.get("latent.heads", (n, H * spec.value_dim), rt.dtype)
        gate = None
        if spec.output_gate:
            gate = packed[:, self.gate_offset:self.gate_offset + (H if spec.head_gate else H * spec.value_dim)]
        ops.head_linear(mixed, self.w_uv, heads, ctx.token_seq, gate=gate, w_rows=self.w_uv_rows, gate_per_head=spec.head_gate)
        y = ws.get("mixer.out", (n, spec.hidden_size), rt.dtype)
        return ops.gemm(heads, self.w_o, y, defer_sum=True) or y
