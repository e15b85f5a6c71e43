"""A plain, slow Zedudra forward pass: one function per mechanism, no paged cache, no kernels.

It imports nothing from the engine and runs on the CPU in the dtype of its inputs (tests use
float64). ``weights`` maps the names on disk (``l0.mix.q``, ``l1.mlp.e3.up`` ...) to tensors; ``cfg``
is the raw dictionary of ``config.json``.

Notation: matrices are stored [out, in] and applied as ``x @ W.T``; a sequence's tokens stand at
positions 0, 1, 2, ... Every function that looks back along the sequence takes and returns what it
has to remember, so that a sequence can be fed in pieces of any size.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional, Tuple

import torch

GATE_SLOPE = 1.702        # g * sigmoid(GATE_SLOPE * g) in an expert


def grouped_rms_norm(x: torch.Tensor, weight: torch.Tensor, groups: int, eps: float) -> torch.Tensor:
    """x [n, w] is cut into ``groups`` equal runs of neighbouring channels; each run is divided by the
    root of (its own mean square + eps); the whole row is then multiplied by ``weight``."""
    n, w = x.shape
    parts = x.reshape(n, groups, w // groups)
    parts = parts / torch.sqrt(parts.pow(2).mean(-1, keepdim=True) + eps)
    return parts.reshape(n, w) * weight


def input_conv(h: torch.Tensor, taps: torch.Tensor, before: Optional[torch.Tensor] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """h [n, c] -> h + conv(h): conv(h)[t] = sum_j taps[:, j] * h[t - (T - 1) + j], the last column of
    ``taps`` [c, T] multiplying the current row. ``before`` [T - 1, c]: the rows in front of h (zeros at
    a sequence's start). Returns (h + conv(h), the last T - 1 rows seen)."""
    n, c = h.shape
    T = taps.shape[1]
    hist = torch.zeros(T - 1, c, dtype=h.dtype) if before is None else before
    ext = torch.cat([hist, h], dim=0)             # row t + T - 1 is h[t]
    y = h.clone()
    for j in range(T):
        y = y + ext[j:j + n] * taps[:, j]
    return y, ext[n:]


def rotate_pairs(x: torch.Tensor, positions: torch.Tensor, dims: int, base: float) -> torch.Tensor:
    """x [n, heads, d]: channels (2i, 2i + 1), i < dims / 2, turn by the angle position * base^(-2i / dims);
    channels from ``dims`` on pass."""
    if dims == 0:
        return x
    i = torch.arange(dims // 2, dtype=x.dtype)
    freq = base ** (-2.0 * i / dims)
    ang = positions.to(x.dtype)[:, None] * freq[None, :]             # [n, dims / 2]
    c, s = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    u, v = x[..., 0:dims:2], x[..., 1:dims:2]
    out = x.clone()
    out[..., 0:dims:2] = u * c - v * s
    out[..., 1:dims:2] = v * c + u * s
    return out


def visible(i: int, j: int, window: int, keep_first: int) -> bool:
    """Whether the query at position i sees the key at position j."""
    return j <= i and (i - j < window or j < keep_first)


def visibility(start: int, n: int, window: int, keep_first: int) -> torch.Tensor:
    """bool [n, start + n]: row t is the query at position start + t, column j the key at position j."""
    i = torch.arange(start, start + n)[:, None]
    j = torch.arange(start + n)[None, :]
    return (j <= i) & ((i - j < window) | (j < keep_first))


def attention_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], prefix: str, m: dict, start: int = 0,
                    past: Optional[Tuple[torch.Tensor, torch.Tensor]] = None, rnd=None):
    """h [n, width]: rows at positions start .. start + n - 1. ``past`` = (rotated keys, values) of the positions
    in front, [start, G, d] each. Returns (output [n, width], (keys, values) of positions 0 .. start + n - 1).
    ``rnd`` rounds what an engine with 16-bit activations stores (projections, cached rows, the gated output)."""
    rnd = rnd or (lambda t: t)
    H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    assert Dv == D, "the values are the keys as projected: they have the keys' size"
    n = h.shape[0]
    pos = torch.arange(start, start + n)
    q = rnd(h @ w[prefix + "q"].T).view(n, H, D)
    k = rnd(h @ w[prefix + "k"].T).view(n, G, D)
    gate = torch.sigmoid(rnd(h @ w[prefix + "g"].T))                 # [n, H]
    v = k                                                            # before the rotation
    rot = m.get("rot") or {"dims": 0, "base": 1.0}
    q = rnd(rotate_pairs(q, pos, rot["dims"], rot["base"]))
    k = rnd(rotate_pairs(k, pos, rot["dims"], rot["base"]))
    if past is not None:
        k = torch.cat([past[0], k], dim=0)
        v = torch.cat([past[1], v], dim=0)
    size, first = m["mask"]["size"], m["mask"].get("keep_first", 0)
    allowed = visibility(start, n, size, first)                      # [n, start + n]
    out = torch.zeros(n, H, Dv, dtype=h.dtype)
    for hd in range(H):
        g = hd // (H // G)
        s = (q[:, hd] @ k[:, g].T) * m["scale"]                      # [n, start + n]
        s = torch.where(allowed, s, torch.full_like(s, float("-inf")))
        out[:, hd] = torch.softmax(s, dim=-1) @ v[:, g]
    out = rnd(out * gate[:, :, None]).reshape(n, H * Dv)
    return out @ w[prefix + "o"].T, (k, v)


def softplus(z: torch.Tensor) -> torch.Tensor:
    return torch.log1p(torch.exp(-z.abs())) + torch.clamp(z, min=0)


def xielu(z: torch.Tensor, p: torch.Tensor, q: torch.Tensor) -> torch.Tensor:
    """z > 0: softplus(p) z^2 + z / 2;  z <= 0: (1/2 + softplus(q)) (exp(z) - 1 - z) + z / 2."""
    a_pos = softplus(p)
    a_neg = 0.5 + softplus(q)
    zn = torch.clamp(z, max=0)
    return torch.where(z > 0, a_pos * z * z + 0.5 * z, a_neg * (torch.expm1(zn) - zn) + 0.5 * z)


def dense_ff(h: torch.Tensor, w: Dict[str, torch.Tensor], prefix: str, rnd=None) -> torch.Tensor:
    rnd = rnd or (lambda t: t)
    act = w[prefix + "act"].to(h.dtype)
    return rnd(xielu(rnd(h @ w[prefix + "up"].T), act[0], act[1])) @ w[prefix + "down"].T


def route(z: torch.Tensor, groups: int, keep: int, top: int) -> Tuple[torch.Tensor, torch.Tensor]:
    """z [n, E] router logits -> (chosen experts [n, top], their weights [n, top]). Scores are sigmoid(z); a
    group of neighbours is worth the sum of its two largest scores (of its one score if it has one); only
    experts of the ``keep`` best groups can be chosen; the weights are the chosen scores as they are."""
    n, E = z.shape
    s = torch.sigmoid(z)
    per = E // groups
    gs = s.view(n, groups, per)
    worth = gs.topk(min(2, per), dim=-1).values.sum(-1)              # [n, groups]
    kept = worth.topk(keep, dim=-1).indices
    allowed = torch.zeros(n, groups, dtype=torch.bool)
    allowed.scatter_(1, kept, True)
    masked = torch.where(allowed[:, :, None].expand(n, groups, per).reshape(n, E), s, torch.full_like(s, -1.0))
    ids = masked.topk(top, dim=-1).indices
    return ids, s.gather(1, ids)


def expert_ff(h: torch.Tensor, gate: torch.Tensor, up: torch.Tensor, down: torch.Tensor, limit: float, rnd=None) -> torch.Tensor:
    """g = min(W_gate h, limit); u = clamp(W_up h, -limit, limit); W_down (g sigmoid(1.702 g) (u + 1))."""
    rnd = rnd or (lambda t: t)
    g = torch.clamp(rnd(h @ gate.T), max=limit)
    u = torch.clamp(rnd(h @ up.T), min=-limit, max=limit)
    return rnd(g * torch.sigmoid(GATE_SLOPE * g) * (u + 1)) @ down.T


def moe_ff(h: torch.Tensor, w: Dict[str, torch.Tensor], prefix: str, f: dict, rnd=None) -> torch.Tensor:
    r = f["router"]
    grp = r.get("groups") or {"count": 1, "keep": 1}
    z = h @ w[prefix + "router"].to(h.dtype).T
    ids, weights = route(z, grp["count"], grp["keep"], r["top"])
    out = torch.zeros_like(h)
    for e in range(r["experts"]):
        rows, which = (ids == e).nonzero(as_tuple=True)
        if rows.numel() == 0:
            continue
        y = expert_ff(h[rows], w[f"{prefix}e{e}.gate"], w[f"{prefix}e{e}.up"], w[f"{prefix}e{e}.down"],
                      f["expert"]["limit"], rnd)
        out[rows] += y * weights[rows, which][:, None]
    return out


def round_to_bfloat16(t: torch.Tensor) -> torch.Tensor:
    return t.to(torch.bfloat16).to(t.dtype)


def weight_layer(cfg: dict, i: int) -> int:
    """The layer whose tensors layer i uses."""
    j = cfg["layers"][i].get("weights_of")
    return i if j is None else j


def forward(cfg: dict, w: Dict[str, torch.Tensor], tokens: List[int], start: int = 0, state: Optional[list] = None,
            rnd=None, layers_out: Optional[list] = None):
    """Logits [n, vocab] of ``tokens`` at positions start .. ; ``state`` is what an earlier call returned for the
    positions in front (None at a sequence's start). Returns (logits, state). ``layers_out`` collects the residual
    stream after every layer."""
    rnd = rnd or (lambda t: t)
    dt = w["embed"].dtype
    eps, groups = cfg["norm"]["eps"], cfg["norm"].get("groups", 1)
    x = w["embed"][torch.tensor(tokens)] * cfg["embedding"]["scale"]
    state = state or [None] * len(cfg["layers"])
    new_state = []
    for i, layer in enumerate(cfg["layers"]):
        p = f"l{weight_layer(cfg, i)}."
        st = state[i] or {}
        h = rnd(grouped_rms_norm(x, w[p + "norm1"], groups, eps))
        conv = None
        if p + "canon1" in w:                        # (a model without the convolution stores no taps)
            h, conv = input_conv(h, w[p + "canon1"], st.get("conv"))
            h = rnd(h)
        y, kv = attention_mixer(h, w, p + "mix.", layer["mixer"], start, st.get("kv"), rnd)
        x = x + grouped_rms_norm(rnd(y), w[p + "norm1b"], groups, eps)
        f = layer.get("mlp")
        if f is not None:
            h = rnd(grouped_rms_norm(x, w[p + "norm2"], groups, eps))
            y = dense_ff(h, w, p + "mlp.", rnd) if f["kind"] == "dense" else moe_ff(h, w, p + "mlp.", f, rnd)
            x = x + grouped_rms_norm(rnd(y), w[p + "norm2b"], groups, eps)
        new_state.append({"conv": conv, "kv": kv})
        if layers_out is not None:
            layers_out.append(x.clone())
    h = rnd(grouped_rms_norm(x, w["final.norm"], groups, eps))
    return h @ w["head"].T, new_state
