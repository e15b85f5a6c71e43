"""Block arrangements: how a layer's norms, mixer and feed-forward are wired.

Reference: minivllm/models/models/qwen3.py:141-156 — norm before the mixer, residual add,
norm before the feed-forward, residual add; nothing after either.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Dict, Optional, Tuple

import torch

from .base import Block, FeedForward, HiddenStream, Mixer, Norm, PartSpec, register_block


@dataclass(frozen=True)
class PreNormBlockSpec(PartSpec):
    kind = "pre_norm"


@register_block(PreNormBlockSpec.kind)
class PreNormBlock(Block):
    """x = x + mixer(norm_mixer(x)); x = x + ffn(norm_ffn(x)). Each residual add is deferred
    into the next norm's kernel through the stream's pending delta."""
    norm_slots: Tuple[str, ...] = ("mixer", "ffn")

    @classmethod
    def slots_for(cls, has_ffn: bool) -> Tuple[str, ...]:
        return cls.norm_slots if has_ffn else cls.norm_slots[:1]

    def __init__(self, spec: PreNormBlockSpec, norms: Dict[str, Norm], mixer: Mixer, ffn: FeedForward):
        self.norm_mixer = norms["mixer"]
        self.norm_ffn = norms.get("ffn")
        if ffn is not None and self.norm_ffn is None:
            raise ValueError("a pre-norm block with a feed-forward needs the norm in front of it")
        self.mixer = mixer
        self.ffn = ffn

    accepts_next_norm = True

    def entry_norm(self) -> Norm:
        return self.norm_mixer

    def entry_part(self):
        return self.mixer

    def forward(self, stream: HiddenStream, ctx, call: int, next_norm: Optional[Norm] = None, next_part=None) -> None:
        # a part that starts with one matrix product over its input may get the norm unrun, to
        # fuse it into that product; a part that ends with one may be offered the add and the norm
        # that follow it, to fold them into that product, when the part behind that norm can go on
        # from rows that are not yet divided by their root mean square
        if self.ffn is None:             # a layer without a feed-forward: the mixer's half alone
            self._run(stream, ctx, self.norm_mixer, self.mixer, next_norm, next_part, (call,))
            return
        self._run(stream, ctx, self.norm_mixer, self.mixer, self.norm_ffn, self.ffn, (call,))
        self._run(stream, ctx, self.norm_ffn, self.ffn, next_norm, next_part, ())

    @staticmethod
    def _run(stream: HiddenStream, ctx, norm: Norm, part, norm_after: Optional[Norm], part_after, extra: tuple) -> None:
        defer = getattr(part, "accepts_pending_norm", False)
        h = norm.pending(stream, ctx) if defer else norm.forward(stream, ctx)
        fold = None
        if norm_after is not None and getattr(part, "accepts_fold", False) \
                and getattr(part_after, "accepts_pending_norm", False):
            make = getattr(norm_after, "fold", None)
            first = getattr(part_after, "first_product", None)
            if make is not None and first is not None:
                fold = make(stream, ctx, first())
        out = part.forward(h, ctx, *extra, fold=fold) if fold is not None else part.forward(h, ctx, *extra)
        if getattr(out, "is_weighted_rows", False):
            stream.delta, stream.weighted = None, out      # already added to the residual
        else:
            stream.delta = out


@dataclass(frozen=True)
class SandwichBlockSpec(PartSpec):
    """A norm in front of and behind every sublayer; ``token_shift`` mixes each row of the mixer's
    input with the row of the token before it (``hidden_size`` is the width of those rows);
    ``input_conv_taps`` > 0 adds to each row of the mixer's input a causal convolution over time of
    those rows, channel by channel, with that many taps."""
    kind = "sandwich"
    hidden_size: int = 0
    token_shift: bool = False
    input_conv_taps: int = 0


@register_block(SandwichBlockSpec.kind)
class SandwichBlock(Block):
    """x = x + norm_mixer_out(mixer(shift(norm_mixer(x)))); x = x + norm_ffn_out(ffn(norm_ffn(x))).

    ``shift``: h[t] <- h[t] + (h[t-1] - h[t]) * mix, element by element, with the rows as the norm
    left them; the row in front of a request's first token is zero, and the last row of a step is
    kept as the request's state (``shift.last``) for its next step. With an input convolution of T
    taps instead: h[t] <- h[t] + sum_j canon[:, j] * h[t - T + 1 + j] (the last tap multiplies h[t]
    itself), zeros in front of a request's first token; the last T - 1 rows are the request's state
    (``conv.last``). A layer without a feed-forward has only the first half.

    The norm behind a sublayer, the residual add and the norm in front of the next sublayer are
    one kernel when both norms are plain scaled RMS norms (``Norm.as_scaled_rms``): the sum never
    leaves float32 and the next norm finds its rows in ``stream.normed``."""
    norm_slots: Tuple[str, ...] = ("norm1", "norm1b", "norm2", "norm2b")
    accepts_next_norm = True
    wants_runtime = True

    @classmethod
    def slots_for(cls, has_ffn: bool) -> Tuple[str, ...]:
        return cls.norm_slots if has_ffn else cls.norm_slots[:2]

    @classmethod
    def tensors(cls, spec: SandwichBlockSpec):
        from .base import TensorDecl
        t = {"shift": TensorDecl((spec.hidden_size,), init="zeros_normal")} if spec.token_shift else {}
        if spec.input_conv_taps > 0:
            t["canon"] = TensorDecl((spec.hidden_size, spec.input_conv_taps), init="zeros_normal")
        return t

    @classmethod
    def state_shapes(cls, spec: SandwichBlockSpec):
        # the mixer's input row of the request's last token, in the activation type (None: the runtime's)
        shapes = {"shift.last": ((spec.hidden_size,), None)} if spec.token_shift else {}
        if spec.input_conv_taps > 1:
            # the mixer's input rows of the request's last taps - 1 tokens, as the norm left them
            shapes["conv.last"] = ((spec.input_conv_taps - 1, spec.hidden_size), None)
        return shapes

    def __init__(self, spec: SandwichBlockSpec, norms: Dict[str, Norm], mixer: Mixer, ffn: FeedForward,
                 tensors=None, rt=None):
        self.spec, self.rt = spec, rt
        self.mixer, self.ffn = mixer, ffn
        self.norm_in, self.norm_out = norms["norm1"], norms["norm1b"]
        self.norm_ffn_in, self.norm_ffn_out = (norms["norm2"], norms["norm2b"]) if ffn is not None else (None, None)
        self.shift = (tensors or {}).get("shift")
        if spec.token_shift and (self.shift is None or rt is None):
            raise ValueError("a block with token shift needs its 'shift' tensor and the runtime")
        self.canon = (tensors or {}).get("canon")
        if spec.input_conv_taps > 0 and (self.canon is None or rt is None):
            raise ValueError("a block with an input convolution needs its 'canon' tensor and the runtime")
        # the same taps tap by tap, [taps, width]: the kernels then read eight channels' weights of a tap in one load
        self.canon_t = self.canon.t().contiguous() if self.canon is not None else None
        if spec.input_conv_taps > 0 and spec.token_shift:
            raise ValueError("a block shapes its mixer's input by a token shift or by a convolution, not both")

    def entry_norm(self) -> Norm:
        return self.norm_in

    def entry_part(self):
        # the rows pass through the shift first: no product takes the norm over; a block in front may
        # apply this block's shift together with its norm (``TokenShiftEntry``)
        if self.canon is not None:
            return InputConvEntry(self.canon, self.canon_t)
        return TokenShiftEntry(self.shift) if self.shift is not None else None

    def _conv_state(self, ctx, call: int):
        return ctx.state(call, "conv.last") if self.spec.input_conv_taps > 1 else None

    def forward(self, stream: HiddenStream, ctx, call: int, next_norm: Optional[Norm] = None, next_part=None) -> None:
        mine = self.shift if self.shift is not None else self.canon
        already = mine is not None and stream.normed is not None and len(stream.normed) > 2 and stream.normed[2] is mine
        h = self.norm_in.forward(stream, ctx)
        if self.shift is not None and not already:
            mixed = self.rt.workspace.get("shift.out", tuple(h.shape), h.dtype)
            self.rt.ops.token_shift(h, self.shift, ctx.state(call, "shift.last"), ctx.token_seq, ctx.cu_seqlens,
                                    ctx.state_slots, mixed)
            h = mixed
        elif self.canon is not None and not already:
            mixed = self.rt.workspace.get("conv.out", tuple(h.shape), h.dtype)
            self.rt.ops.input_conv(h, self.canon, self._conv_state(ctx, call), ctx.token_seq, ctx.cu_seqlens,
                                   ctx.state_slots, ctx.n_seqs, mixed, taps_t=self.canon_t)
            h = mixed
        y = self.mixer.forward(h, ctx, call)
        last = self.ffn is None
        self._close(stream, ctx, y, self.norm_out, next_norm if last else self.norm_ffn_in, call, next_part if last else None)
        if not last:
            h = self.norm_ffn_in.forward(stream, ctx)
            y = self.ffn.forward(h, ctx)
            self._close(stream, ctx, y, self.norm_ffn_out, next_norm, call, next_part)

    def _close(self, stream: HiddenStream, ctx, y, norm_out: Norm, norm_next: Optional[Norm], call: int = 0,
               next_part=None) -> None:
        """resid += norm_out(y); the rows of ``norm_next`` are left in the stream when it can ride along, and
        in a step of single tokens the next block's token shift with them."""
        if not isinstance(y, torch.Tensor):
            y = y.materialize()
        out_form = norm_out.as_scaled_rms()
        next_form = norm_next.as_scaled_rms() if norm_next is not None else None
        if out_form is None and self._close_grouped(stream, ctx, y, norm_out, norm_next, call, next_part):
            return
        if out_form is None:
            tmp = self.rt.workspace.get("sandwich.delta", tuple(y.shape), y.dtype)
            norm_out.apply(y, tmp)
            stream.delta = tmp           # the next norm (or the model's last) adds it
            return
        rows = None
        if next_form is not None:
            rows = self.rt.workspace.get("normed", tuple(y.shape), y.dtype)
        shift = None
        plan = getattr(ctx, "attention_plan", None)
        if rows is not None and isinstance(next_part, TokenShiftEntry) and plan is not None and plan.decode_only:
            # the block that runs next is call + 1: its shift state is that call's
            shift = (next_part.mix, ctx.state(call + 1, "shift.last"), ctx.token_seq, ctx.state_slots)
        self.rt.ops.norm_add_norm(y, out_form, stream.resid, next_form, rows, shift=shift)
        stream.delta = None
        if rows is None:
            stream.normed = None
        else:
            stream.normed = (norm_next, rows, next_part.mix) if shift is not None else (norm_next, rows)


    def _close_grouped(self, stream: HiddenStream, ctx, y, norm_out: Norm, norm_next: Optional[Norm], call: int,
                       next_part) -> bool:
        """The same in one kernel for norms in groups (``as_grouped_rms``); in a step of single tokens the next
        block's input convolution rides along. False, having done nothing, when the norms are of another form."""
        form = getattr(norm_out, "as_grouped_rms", None)
        if form is None:
            return False
        wa, eps_a, groups = form()
        nxt = getattr(norm_next, "as_grouped_rms", None) if norm_next is not None else None
        rows = second = conv = None
        if nxt is not None and nxt()[2] == groups:
            wb, eps_b, _ = nxt()
            second = (wb, eps_b)
            rows = self.rt.workspace.get("normed", tuple(y.shape), y.dtype)
        plan = getattr(ctx, "attention_plan", None)
        if rows is not None and isinstance(next_part, InputConvEntry) and plan is not None and plan.decode_only:
            taps = next_part.taps
            state = ctx.state(call + 1, "conv.last") if taps.shape[1] > 1 else None    # the block that runs next is call + 1
            conv = (taps, state, ctx.token_seq, ctx.state_slots, next_part.taps_t)
        self.rt.ops.group_norm_add_norm(y, (wa, eps_a), stream.resid, second, rows, groups, conv=conv)
        stream.delta = None
        if rows is None:
            stream.normed = None
        else:
            stream.normed = (norm_next, rows, next_part.taps) if conv is not None else (norm_next, rows)
        return True


class InputConvEntry:
    """What a sandwich block with an input convolution offers the block in front of it: the taps, so that
    its rows can leave that block's last kernel with the convolution applied."""

    def __init__(self, taps: torch.Tensor, taps_t: Optional[torch.Tensor] = None):
        self.taps, self.taps_t = taps, taps_t


class TokenShiftEntry:
    """What a sandwich block with a token shift offers the block in front of it: the shift's weights, so
    that its rows can leave that block's last kernel already shifted."""

    def __init__(self, mix: torch.Tensor):
        self.mix = mix


@dataclass(frozen=True)
class HyperConnectionBlockSpec(PartSpec):
    """Pre-norm sublayers on ``streams`` residual streams of width ``hidden_size`` instead of one."""
    kind = "hyper_connections"
    hidden_size: int = 0
    streams: int = 1
    has_ffn: bool = True            # a layer without a feed-forward has no second set of stream weights


class HyperEntry:
    """What a block on several residual streams offers the block in front of it: its first sublayer's read,
    so that a block of the same kind can leave its last write to that read's kernel."""

    def __init__(self, block: "HyperConnectionBlock"):
        self.block = block


@register_block(HyperConnectionBlockSpec.kind)
class HyperConnectionBlock(Block):
    """A token's residual is S streams x_1 .. x_S, all equal to the embedding's output in front of the first
    layer. Sublayer q (1: mixer, 2: feed-forward) with its stored weights ``hc<q>.in`` [S], ``hc<q>.out`` [S]
    and ``hc<q>.mix`` [S, S] (indexed [from, to]):

        u = sum_s in[s] x_s;   y = sublayer(norm_q(u));   x_t <- sum_s mix[s, t] x_s + out[t] y   (all t at once)

    Behind the last layer the streams are summed into the plain residual. The streams live in
    ``HiddenStream.lanes`` (float32); a write waits in ``lanes_write`` for the kernel of the next read, so
    the streams are read and written once between two sublayers (``ops.hyper_step``). The norms must be
    plain scaled RMS norms: the read's kernel applies them itself."""
    norm_slots: Tuple[str, ...] = ("norm1", "norm2")
    accepts_next_norm = True
    wants_runtime = True

    @classmethod
    def slots_for(cls, has_ffn: bool) -> Tuple[str, ...]:
        return cls.norm_slots if has_ffn else cls.norm_slots[:1]

    @classmethod
    def tensors(cls, spec: HyperConnectionBlockSpec):
        from .base import TensorDecl
        S = spec.streams
        t = {}
        for q in ((1, 2) if spec.has_ffn else (1,)):
            t[f"hc{q}.in"] = TensorDecl((S,), init="ones_normal")
            t[f"hc{q}.out"] = TensorDecl((S,), init="ones_normal")
            t[f"hc{q}.mix"] = TensorDecl((S, S), init="identity_normal")
        return t

    def __init__(self, spec: HyperConnectionBlockSpec, norms: Dict[str, Norm], mixer: Mixer, ffn: FeedForward,
                 tensors=None, rt=None):
        if rt is None or tensors is None:
            raise ValueError("a block on several residual streams needs its tensors and the runtime")
        if spec.streams < 1 or spec.streams > 8:
            raise ValueError(f"1 to 8 residual streams are served, got {spec.streams}")
        self.spec, self.rt, self.mixer, self.ffn = spec, rt, mixer, ffn
        self.sublayers = []
        for q, part in ((1, mixer), (2, ffn)):
            if part is None:
                continue
            form = norms[f"norm{q}"].as_scaled_rms()
            if form is None or form[2]:
                raise ValueError("the norms of a block on several residual streams must be plain scaled RMS norms")
            # the residual sum is float32 whatever type the weights are stored in
            w = {k: tensors[f"hc{q}.{k}"].to(torch.float32).contiguous() for k in ("in", "out", "mix")}
            self.sublayers.append((part, w, form[0], form[1]))

    def entry_norm(self) -> Optional[Norm]:
        return None                     # the read applies it: no product may take it over

    def entry_part(self):
        return HyperEntry(self)

    def forward(self, stream: HiddenStream, ctx, call: int, next_norm: Optional[Norm] = None, next_part=None) -> None:
        rt, ops, spec = self.rt, self.rt.ops, self.spec
        n = stream.resid.shape[0]
        first = None
        if stream.lanes is None:
            if stream.delta is not None:
                raise RuntimeError("a block on several residual streams cannot take a stream with a pending delta")
            stream.lanes = rt.workspace.get("hyper.lanes", (spec.streams, n, spec.hidden_size), torch.float32)
            first = stream.resid
        for index, (part, w, norm_weight, eps) in enumerate(self.sublayers):
            h = rt.workspace.get("normed", (n, spec.hidden_size), rt.dtype)
            ops.hyper_step(stream.lanes, out=h, first=first, write=stream.lanes_write, read=(w["in"], norm_weight, eps))
            first, stream.lanes_write = None, None
            y = part.forward(h, ctx, call) if index == 0 and part is self.mixer else part.forward(h, ctx)
            if not isinstance(y, torch.Tensor):
                y = y.materialize()
            stream.lanes_write = (y, w["mix"], w["out"])
        if not isinstance(next_part, HyperEntry):
            self.close_stream(stream, ctx)

    def close_stream(self, stream: HiddenStream, ctx) -> None:
        """The last write and the sum of the streams: ``stream.resid`` is the plain residual again."""
        if stream.lanes is None:
            return
        self.rt.ops.hyper_step(stream.lanes, write=stream.lanes_write, total=stream.resid)
        stream.lanes, stream.lanes_write, stream.delta = None, None, None
