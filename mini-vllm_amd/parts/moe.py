"""A mixture of gated feed-forward experts behind a softmax router.

Router logits z = W_router x in float32; scores s = softmax(z) over all router outputs. The last
``identity_experts`` outputs are identity experts (their output is x itself, they have no tensors), the
others are gated SiLU pairs down_e(silu(gate_e x) * (up_e x)). A token uses ``top`` experts: those with
the largest s + correction (the correction steers the choice only, never the weights), restricted to
the ``keep_groups`` of ``groups`` equal runs of neighbouring router outputs whose largest such number is
largest (outputs of other groups cannot be chosen whatever their number). The weights are the chosen
experts' scores divided by their sum (+ weight_sum_eps); the result is the weighted sum of the
chosen experts' outputs.

How it runs: gate and up matrices of all experts form one packed product and all down matrices one
second product; between them one kernel applies SiLU, the up factor and the router's weight (zero
for experts that were not chosen) before the single rounding, so the second product sums exactly the
chosen experts. That is exact, replays from graphs and runs at the library product's rate, but computes
every expert: eight times the useful multiply-adds when a token uses an eighth of the experts, and every
expert's bytes in a decode step. With ``grouped`` (bfloat16, widths that are multiples of 32) the chosen
(token, expert) pairs are instead sorted by expert on the device, every expert's pairs are cut into tiles
of 64 rows, and two MFMA kernels compute gate/up with the weighted activation and the down product for
those tiles only; a last kernel sums a token's pairs in the order of choice and adds the identity experts'
share. Its plain MFMA kernels (operands straight from memory) win where bytes decide, steps of few rows
against large experts (8B-sized layers, 32 experts, 4 a token: a step of one request 8.8 against 13.1 ms,
of eight 12.2 against 13.4), and lose or draw elsewhere (0.6B-sized layers at eight requests 3.0 against
2.4 ms; a prompt of 2,048 tokens 440 against 465 us a layer at 0.6B sizes, but 186 against 151 ms for the
whole prompt at 8B sizes), so the spec's thresholds send only the former there. Either way everything is decided on the device;
nothing about a step's routing reaches the host, so steps replay from graphs.

Options of the spec, each with the default that gives the above: ``scoring`` "sigmoid" scores every router
output by sigmoid(z) on its own; ``group_worth`` "top2" ranks a group by the sum of its two largest choices
instead of its largest; ``normalize`` False uses the chosen scores themselves as weights; ``activation``
"clamped" replaces the gated SiLU pair by g = min(gate, limit), u = clamp(up, -limit, limit),
g * sigmoid(gate_slope * g) * (u + 1).

``router`` "table": there is no router. A stored integer table [``table_rows``, ``top``] names the experts of every
token id (the step's ``ctx.token_ids``), each with the weight 1 / top; with all experts at once the activation kernel
looks the weights up itself, the chosen-pairs path gets the usual lists from ``moe_table_route``. ``shared_size`` > 0:
a shared expert (a gated pair like the others) runs for every token and is added: its rows ride in the two packed
products, or, where steps may take the chosen pairs only, it keeps two products of its own.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict

import torch

from .base import FeedForward, PartSpec, Runtime, TensorDecl, register_feed_forward


@dataclass(frozen=True)
class RoutedExpertsSpec(PartSpec):
    kind = "routed_swiglu"
    hidden_size: int = 0
    expert_size: int = 0                 # width of one expert's gated pair
    num_experts: int = 0                 # experts with tensors
    identity_experts: int = 0            # router outputs behind them whose expert is the identity
    top: int = 1
    groups: int = 1
    keep_groups: int = 1
    correction: bool = False             # a stored number per router output added to the scores for the choice
    weight_sum_eps: float = 1e-20
    # bfloat16, widths that are multiples of 32: the experts' products over the chosen (token, expert) pairs only, in steps
    # with fewer than ``grouped_max_rows`` chosen rows an expert on average and experts of at least ``grouped_min_weight``
    # elements a matrix (there a step is bound by the bytes of the experts it reads, and most experts are not chosen)
    grouped: bool = True
    grouped_max_rows: float = 2.0
    grouped_min_weight: int = 4 * 1024 * 1024
    scoring: str = "softmax"             # or "sigmoid"
    group_worth: str = "max"             # or "top2": the sum of a group's two largest choices
    normalize: bool = True               # False: the weights are the chosen scores as they are
    activation: str = "swiglu"           # or "clamped" (with ``limit`` and ``gate_slope``)
    limit: float = 0.0
    gate_slope: float = 1.702
    # "table": no router product; a stored integer table [table_rows, top] names the experts of every token id, each
    # with the weight 1 / top (``groups``, ``correction``, ``scoring`` and ``normalize`` then mean nothing)
    router: str = "learned"
    table_rows: int = 0
    # > 0: a shared expert of that width (a gated pair like the others) runs for every token and is added
    shared_size: int = 0

    @property
    def router_outputs(self) -> int:
        return self.num_experts + self.identity_experts


@register_feed_forward(RoutedExpertsSpec.kind)
class RoutedExperts(FeedForward):
    spec_class = RoutedExpertsSpec

    @classmethod
    def tensors(cls, spec: RoutedExpertsSpec) -> Dict[str, TensorDecl]:
        if spec.router == "table":
            t = {"table": TensorDecl((spec.table_rows, spec.top), init=f"distinct_below:{spec.num_experts}", integer=True)}
        else:
            t = {"router": TensorDecl((spec.router_outputs, spec.hidden_size))}
        if spec.shared_size:
            t["shared.gate"] = TensorDecl((spec.shared_size, spec.hidden_size))
            t["shared.up"] = TensorDecl((spec.shared_size, spec.hidden_size))
            t["shared.down"] = TensorDecl((spec.hidden_size, spec.shared_size))
        if spec.correction:
            t["correction"] = TensorDecl((spec.router_outputs,), init="zeros_normal")
        for e in range(spec.num_experts):
            t[f"gate.{e}"] = TensorDecl((spec.expert_size, spec.hidden_size))
            t[f"up.{e}"] = TensorDecl((spec.expert_size, spec.hidden_size))
            t[f"down.{e}"] = TensorDecl((spec.hidden_size, spec.expert_size))
        return t

    def __init__(self, spec: RoutedExpertsSpec, tensors: Dict[str, torch.Tensor], rt: Runtime):
        E = spec.router_outputs
        if spec.num_experts < 0 or spec.identity_experts < 0 or E < 1 or spec.groups < 1 or E % spec.groups \
                or not (1 <= spec.keep_groups <= spec.groups) or not (1 <= spec.top <= E // spec.groups * spec.keep_groups):
            raise ValueError(f"routed experts: bad sizes {spec}")
        if spec.scoring not in ("softmax", "sigmoid") or spec.group_worth not in ("max", "top2") \
                or spec.activation not in ("swiglu", "clamped") or (spec.activation == "clamped" and not spec.limit > 0):
            raise ValueError(f"routed experts: unknown scoring, group worth or activation, or a clamped pair without a "
                             f"positive limit: {spec}")
        if spec.router not in ("learned", "table") or spec.shared_size < 0:
            raise ValueError(f"routed experts: the router is 'learned' or 'table' and a shared expert's width >= 0: {spec}")
        if spec.router == "table" and (spec.identity_experts or spec.correction or spec.table_rows < 1 or not spec.num_experts):
            raise ValueError(f"routed experts: a table names experts with tensors, for every token id: {spec}")
        if spec.shared_size and not spec.num_experts:
            raise ValueError("routed experts: a shared expert stands beside experts with tensors")
        self.spec, self.rt = spec, rt
        self.w_router = tensors.get("router")
        self.table = tensors.get("table")
        self.correction = tensors.get("correction")
        n_e = spec.num_experts
        if n_e:
            names = [f"{k}.{e}" for e in range(n_e) for k in ("gate", "up", "down")]
            if spec.shared_size:
                names += ["shared.gate", "shared.up", "shared.down"]
            dtypes = {tensors[name].dtype for name in names}
            if len(dtypes) != 1:
                raise ValueError(f"routed experts: the experts are stored in different dtypes {dtypes}; cannot pack them")
            # rows: every expert's gate block, then every expert's up block; the down matrices side by side. A shared
            # expert's gate and up rows come behind those and its down matrix behind the others' (one pair of products
            # serves all), unless steps may take the chosen pairs only: then it keeps matrices and products of its own
            self.shared_packed = bool(spec.shared_size) and not self._grouped_possible()
            shared_rows = [tensors["shared.gate"], tensors["shared.up"]] if spec.shared_size else []
            self.w_gate_up = torch.cat([tensors[f"gate.{e}"] for e in range(n_e)] + [tensors[f"up.{e}"] for e in range(n_e)]
                                       + (shared_rows if self.shared_packed else []), dim=0).contiguous()
            self.w_down = torch.cat([tensors[f"down.{e}"] for e in range(n_e)]
                                    + ([tensors["shared.down"]] if self.shared_packed else []), dim=1).contiguous()
            if spec.shared_size and not self.shared_packed:
                self.w_shared_gate_up = torch.cat(shared_rows, dim=0).contiguous()
                self.w_shared_down = tensors["shared.down"]

    def _grouped_possible(self) -> bool:
        spec = self.spec
        return (spec.grouped and self.rt.ops.use_fast_kernels and self.rt.dtype == torch.bfloat16
                and spec.expert_size * spec.hidden_size >= spec.grouped_min_weight)

    def wants_grouped(self, n: int) -> bool:
        """Whether a step of n rows computes the chosen pairs only (where the kernels take the sizes)."""
        spec = self.spec
        return (spec.grouped and n * spec.top < spec.grouped_max_rows * spec.num_experts
                and spec.expert_size * spec.hidden_size >= spec.grouped_min_weight)

    def _grouped(self, x: torch.Tensor, ctx, dense, ids, weights, y) -> bool:
        """The chosen (token, expert) pairs only: sorted by expert on the device, tiles of 64 rows through MFMA.
        False: the sizes are not served."""
        spec, rt, ops, ws = self.spec, self.rt, self.rt.ops, self.rt.workspace
        n, n_e, F = x.shape[0], spec.num_experts, spec.expert_size
        need = int(ops.lib.dll.mv_moe_grouped_ints(n, spec.top, n_e)) if ops.lib.has("mv_moe_grouped") else 0
        return bool(need) and ops.moe_grouped(
            x, self.w_gate_up, self.w_down, n_e, spec.identity_experts, F, ids, weights, dense,
            ws.get("moe.ints", (need,), torch.int32), ws.get("moe.pair_act", (n * spec.top, F), rt.dtype),
            ws.get("moe.pair_out", (n * spec.top, spec.hidden_size), torch.float32), y,
            limit=spec.limit if spec.activation == "clamped" else 0.0, slope=spec.gate_slope)

    def _add_shared(self, x: torch.Tensor, y: torch.Tensor) -> None:
        """y += the shared expert's output, as two products of its own."""
        spec, rt, ops, ws = self.spec, self.rt, self.rt.ops, self.rt.workspace
        n, FS = x.shape[0], spec.shared_size
        if spec.activation != "swiglu":
            raise NotImplementedError("a shared expert with matrices of its own is a gated SiLU pair")
        act = ws.get("moe.shared_act", (n, FS), rt.dtype)
        if not ops.gemm_swiglu(x, self.w_shared_gate_up, act):
            gu = ws.get("moe.shared_gate_up", (n, 2 * FS), rt.dtype)
            ops.gemm(x, self.w_shared_gate_up, gu)
            ops.swiglu(gu, act)
        ys = ws.get("moe.shared_out", (n, spec.hidden_size), rt.dtype)
        ops.gemm(act, self.w_shared_down, ys)
        ops.add_rows(y, ys)

    def forward(self, x: torch.Tensor, ctx) -> torch.Tensor:
        spec, rt, ops, ws = self.spec, self.rt, self.rt.ops, self.rt.workspace
        if not isinstance(x, torch.Tensor):
            x = x.materialize()
        n, E, n_e, F = x.shape[0], spec.router_outputs, spec.num_experts, spec.expert_size
        FS = spec.shared_size if n_e and self.shared_packed else 0
        apart = bool(spec.shared_size) and not FS
        dense = ws.get("moe.dense", (n, E), torch.float32)
        ids = ws.get("moe.ids", (n, spec.top), torch.int32)
        weights = ws.get("moe.weights", (n, spec.top), torch.float32)
        by_table = spec.router == "table"
        grouped = bool(n_e) and ops.use_fast_kernels and self.wants_grouped(n)
        if by_table and grouped:
            ops.moe_table_route(ctx.token_ids, self.table, n_e, dense, ids, weights)
        elif by_table:
            pass                  # all experts at once: the activation kernel looks the weights up itself
        else:
            logits = ws.get("moe.logits", (n, E), torch.float32)
            ops.gemm(x, self.w_router, logits)
            ops.moe_route(logits, self.correction, spec.groups, spec.keep_groups, spec.top, spec.weight_sum_eps, dense, ids, weights,
                          scoring=spec.scoring, group_worth=spec.group_worth, normalize=spec.normalize)
        y = ws.get("ffn.out", (n, spec.hidden_size), rt.dtype)
        if grouped and self._grouped(x, ctx, dense, ids, weights, y):
            if apart:
                self._add_shared(x, y)
            return y
        if grouped and by_table:
            grouped = False       # the sizes were not served after all: the lists are there, the kernel below takes the table
        if n_e:
            gu = ws.get("moe.gate_up", (n, 2 * n_e * F + 2 * FS), rt.dtype)
            ops.gemm(x, self.w_gate_up, gu)
            act = ws.get("moe.act", (n, n_e * F + FS), rt.dtype)
            table = (ctx.token_ids, self.table) if by_table else None
            if spec.activation == "clamped":
                ops.moe_swiglu_scale(gu, None if by_table else dense, n_e, F, act, limit=spec.limit, slope=spec.gate_slope,
                                     shared=FS, table=table)
            else:
                ops.moe_swiglu_scale(gu, None if by_table else dense, n_e, F, act, shared=FS, table=table)
            ops.gemm(act, self.w_down, y)
            if apart:
                self._add_shared(x, y)
        if spec.identity_experts or not n_e:
            ops.moe_identity_add(y, x, dense, n_e, spec.identity_experts, overwrite=not n_e)
        return y
