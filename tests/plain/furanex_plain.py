"""A plain, slow Furanex forward pass: one function per mechanism, no paged cache, no kernels.

It imports nothing from the engine and runs on the CPU in the dtype of its inputs (tests use
float64). ``weights`` maps the names on disk (``l0.mix.q``, ``l1.mlp.e3.up``, ``l2.hc1.mix`` ...) to
tensors; ``cfg`` is the raw dictionary of ``config.json``.

Notation: matrices are stored [out, in] and applied as ``x @ W.T``; a sequence's tokens stand at
positions 0, 1, 2, ... Every function that looks back along the sequence takes and returns what it
has to remember (``past``), so that a sequence can be fed in pieces of any size.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional, Tuple

import torch


def unit_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x divided by the root of (its mean square over the last axis + eps)."""
    return x / torch.sqrt(x.pow(2).mean(-1, keepdim=True) + eps)


def rms_norm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    return unit_rms(x, eps) * weight


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


# ---------------------------------------------------------------------------------------
# Rotation by position, with stretched low frequencies
# ---------------------------------------------------------------------------------------
def rotation_frequencies(dims: int, base: float, scaling: Optional[dict]) -> Tuple[List[float], float]:
    """(frequency of pair i for i < dims / 2, the factor on every cosine and sine).

    Plain: f_i = base^(-2i / dims), factor 1. With ``scaling`` = {factor, original, fast, slow}: a pair
    that turns ``t`` times over ``original`` positions has index d(t) = dims ln(original / (2 pi t)) /
    (2 ln base); between lo = d(fast) (rounded down, at least 0) and hi = d(slow) (rounded up, at most
    dims - 1) a ramp r_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1) blends f_i (r = 0) into
    f_i / factor (r = 1); cosines and sines are multiplied by 0.1 ln(factor) + 1."""
    f = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    if not scaling:
        return f, 1.0
    factor, original = float(scaling["factor"]), float(scaling["original"])

    def index_of(turns: float) -> float:
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(index_of(float(scaling["fast"]))), 0)
    hi = min(math.ceil(index_of(float(scaling["slow"]))), dims - 1)
    out = []
    for i, fi in enumerate(f):
        r = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
        out.append(fi / factor * r + fi * (1.0 - r))
    return out, 0.1 * math.log(factor) + 1.0


def rotate(x: torch.Tensor, positions: torch.Tensor, dims: int, freqs: List[float], factor: float,
           neighbours: bool) -> torch.Tensor:
    """x [n, heads, d]: the first ``dims`` channels of every head turn by position * freqs[i]; the pair i is
    (i, i + dims / 2), or (2i, 2i + 1) with ``neighbours``. The pair (u, v) becomes
    (u c - v s, v c + u s) with c = factor cos, s = factor sin. Channels from ``dims`` on pass."""
    if dims == 0:
        return x
    half = dims // 2
    ang = positions.to(x.dtype)[:, None] * torch.tensor(freqs, dtype=x.dtype)[None, :]
    c, s = (factor * torch.cos(ang))[:, None, :], (factor * torch.sin(ang))[:, None, :]
    out = x.clone()
    if neighbours:
        u, v = x[..., 0:dims:2], x[..., 1:dims:2]
        out[..., 0:dims:2] = u * c - v * s
        out[..., 1:dims:2] = v * c + u * s
    else:
        u, v = x[..., :half], x[..., half:dims]
        out[..., :half] = u * c - v * s
        out[..., half:dims] = v * c + u * s
    return out


def causal_softmax(scores: torch.Tensor, start: int) -> torch.Tensor:
    """scores [..., n, start + n]: row t is the query at position start + t; keys behind it weigh nothing."""
    n, total = scores.shape[-2], scores.shape[-1]
    i = torch.arange(start, start + n)[:, None]
    j = torch.arange(total)[None, :]
    return torch.softmax(scores.masked_fill(j > i, float("-inf")), dim=-1)


# ---------------------------------------------------------------------------------------
# Mixers
# ---------------------------------------------------------------------------------------
def attention_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], prefix: str, m: dict, eps: float, start: int = 0,
                    past=None, first_values: Optional[torch.Tensor] = None, mixes: bool = False, rnd=None):
    """Grouped softmax attention. h [n, width] are the rows at positions start .. start + n - 1; ``past`` =
    (keys, values) of the positions in front, [start, G, d] and [start, G, dv]. q and k are rotated over
    their first ``rot.dims`` channels in half-split pairs and then divided by their root mean square per
    head. With ``mixes`` the values become (1 - l) v + l ``first_values`` (l = the layer's ``vmix``) before
    they are kept. Returns (output [n, width], (keys, values) up to start + n - 1, this step's values [n, G, dv]
    as they were projected)."""
    rnd = rnd or (lambda t: t)
    H, G, D = m["heads"], m.get("kv_heads", m["heads"]), m["dim"]
    Dv = m.get("vdim", D)
    n = h.shape[0]
    q = rnd(h @ w[prefix + "q"].T).reshape(n, H, D)
    k = rnd(h @ w[prefix + "k"].T).reshape(n, G, D)
    v = rnd(h @ w[prefix + "v"].T).reshape(n, G, Dv)
    projected = v
    rot = m.get("rot")
    if rot:
        freqs, factor = rotation_frequencies(rot["dims"], rot["base"], rot.get("scaling"))
        pos = torch.arange(start, start + n)
        q = rotate(q, pos, rot["dims"], freqs, factor, neighbours=False)
        k = rotate(k, pos, rot["dims"], freqs, factor, neighbours=False)
    q, k = unit_rms(q, eps), rnd(unit_rms(k, eps))
    if mixes:
        lam = w[prefix + "vmix"].to(h.dtype)
        v = (1.0 - lam) * v + lam * first_values
    v = rnd(v)
    if past is not None:
        k, v = torch.cat([past[0], k], dim=0), torch.cat([past[1], v], dim=0)
    rep = H // G
    kh, vh = k.repeat_interleave(rep, dim=1), v.repeat_interleave(rep, dim=1)       # head h reads group h // rep
    scores = torch.einsum("nhd,mhd->hnm", q, kh) * m["scale"]
    p = causal_softmax(scores, start)
    o = rnd(torch.einsum("hnm,mhd->nhd", p, vh).reshape(n, H * Dv))
    return rnd(o @ w[prefix + "o"].T), (k, v), projected


def latent_attention_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], prefix: str, m: dict, eps: float, start: int = 0,
                           past=None, rnd=None):
    """Attention whose keys and values are maps of one latent per token. ``past`` = (latents [start, kv_rank],
    rotated key parts [start, rot_dim]). A head's query is [dim plain | rot_dim rotated]; the key part that is
    rotated is one for all heads; rotation in neighbouring pairs. Head h's output is multiplied by
    sigmoid(W_g h)[h]. Returns (output, (latents, key parts) up to start + n - 1)."""
    rnd = rnd or (lambda t: t)
    H, D, Dr, Dv, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    n = h.shape[0]
    cq = rnd(rms_norm(rnd(h @ w[prefix + "dq"].T), w[prefix + "dq.norm"], eps))
    q = rnd(cq @ w[prefix + "uq"].T).reshape(n, H, D + Dr)
    down = rnd(h @ w[prefix + "dkv"].T)
    c = rnd(rms_norm(down[:, :R], w[prefix + "dkv.norm"], eps))
    kr = down[:, R:].reshape(n, 1, Dr)
    rot = m.get("rot")
    pos = torch.arange(start, start + n)
    q_plain, q_rot = q[..., :D], q[..., D:]
    if Dr:
        freqs, factor = rotation_frequencies(Dr, rot["base"], rot.get("scaling"))
        q_rot = rotate(q_rot, pos, Dr, freqs, factor, neighbours=True)
        kr = rotate(kr, pos, Dr, freqs, factor, neighbours=True)
    kr = rnd(kr.reshape(n, Dr))
    if past is not None:
        c, kr = torch.cat([past[0], c], dim=0), torch.cat([past[1], kr], dim=0)
    k_plain = (c @ w[prefix + "uk"].T).reshape(-1, H, D)
    v = (c @ w[prefix + "uv"].T).reshape(-1, H, Dv)
    scores = (torch.einsum("nhd,mhd->hnm", q_plain, k_plain) + torch.einsum("nhd,md->hnm", q_rot, kr)) * m["scale"]
    p = causal_softmax(scores, start)
    o = torch.einsum("hnm,mhd->nhd", p, v)
    gate = torch.sigmoid(h @ w[prefix + "g"].T)                   # [n, H]
    o = rnd((o * gate[:, :, None]).reshape(n, H * Dv))
    return rnd(o @ w[prefix + "o"].T), (c, kr)


# ---------------------------------------------------------------------------------------
# Feed-forward: experts looked up by token id, beside a shared expert
# ---------------------------------------------------------------------------------------
def expert(h: torch.Tensor, w: Dict[str, torch.Tensor], prefix: str, rnd=None) -> torch.Tensor:
    rnd = rnd or (lambda t: t)
    a = rnd(silu(h @ w[prefix + "gate"].T) * (h @ w[prefix + "up"].T))
    return a @ w[prefix + "down"].T


def table_mixture(h: torch.Tensor, tokens: torch.Tensor, w: Dict[str, torch.Tensor], prefix: str, f: dict, rnd=None) -> torch.Tensor:
    """Row t uses the experts ``table[tokens[t]]`` (``top`` of them, each weighing 1 / top); the shared
    expert, where the layer has one, runs for every row and is added."""
    top = f["router"]["top"]
    table = w[prefix + "table"]
    y = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e in table[int(tokens[t])].tolist():
            y[t] = y[t] + expert(h[t:t + 1], w, f"{prefix}e{int(e)}.", rnd)[0] / top
    if f.get("shared"):
        y = y + expert(h, w, prefix + "shared.", rnd)
    return (rnd or (lambda t: t))(y)


# ---------------------------------------------------------------------------------------
# Several residual streams
# ---------------------------------------------------------------------------------------
def streams_read(xs: torch.Tensor, w_in: torch.Tensor) -> torch.Tensor:
    """xs [S, n, width] -> sum_s w_in[s] xs[s]."""
    return torch.einsum("s,snw->nw", w_in.to(xs.dtype), xs)


def streams_write(xs: torch.Tensor, y: torch.Tensor, w_mix: torch.Tensor, w_out: torch.Tensor) -> torch.Tensor:
    """New stream t = sum_s w_mix[s, t] xs[s] + w_out[t] y, all from the old streams."""
    return torch.einsum("st,snw->tnw", w_mix.to(xs.dtype), xs) + w_out.to(xs.dtype)[:, None, None] * y[None]


# ---------------------------------------------------------------------------------------
# The model
# ---------------------------------------------------------------------------------------
def first_mixing_layer(cfg: dict) -> Optional[int]:
    for i, layer in enumerate(cfg["layers"]):
        if layer["type"] == "attention" and layer["mixer"].get("v_mix"):
            return i
    return None


def forward(cfg: dict, w: Dict[str, torch.Tensor], tokens: List[int], start: int = 0, past: Optional[list] = None,
            rnd=None, layer_sums: Optional[list] = None):
    """Logits [n, vocab] of ``tokens`` standing at positions start ...; ``past`` is what an earlier call
    returned for the positions in front. Returns (logits, past). ``layer_sums`` collects the sum of the
    streams behind every layer."""
    dt = w["embed"].dtype
    eps = cfg["norm"]["eps"]
    S = cfg.get("streams")
    ids = torch.tensor(tokens, dtype=torch.long)
    x = w["embed"][ids] * (cfg.get("embedding") or {}).get("scale", 1.0)
    xs = x[None].repeat(S, 1, 1) if S else None
    past = past if past is not None else [None] * len(cfg["layers"])
    new_past = []
    first = first_mixing_layer(cfg)
    first_values = None

    def sublayer(q: int, i: int, fn):
        nonlocal x, xs
        if S:
            u = streams_read(xs, w[f"l{i}.hc{q}.in"])
            y = fn(rms_norm(u, w[f"l{i}.norm{q}"], eps))
            xs = streams_write(xs, y.to(dt), w[f"l{i}.hc{q}.mix"], w[f"l{i}.hc{q}.out"])
        else:
            x = x + fn(rms_norm(x, w[f"l{i}.norm{q}"], eps))

    for i, layer in enumerate(cfg["layers"]):
        m, kept = layer["mixer"], [None]

        def mix(hh, i=i, m=m, layer=layer, kept=kept):
            nonlocal first_values
            hh = (rnd or (lambda t: t))(hh)
            if layer["type"] == "attention":
                mixes = bool(m.get("v_mix")) and i != first
                y, kept[0], projected = attention_mixer(hh, w, f"l{i}.mix.", m, eps, start, past[i], first_values, mixes, rnd)
                if i == first:
                    first_values = projected
                return y
            if layer["type"] == "latent_attention":
                y, kept[0] = latent_attention_mixer(hh, w, f"l{i}.mix.", m, eps, start, past[i], rnd)
                return y
            raise ValueError(layer["type"])

        sublayer(1, i, mix)
        new_past.append(kept[0])
        if layer.get("mlp"):
            sublayer(2, i, lambda hh, i=i, layer=layer: table_mixture((rnd or (lambda t: t))(hh), ids, w, f"l{i}.mlp.", layer["mlp"], rnd))
        if layer_sums is not None:
            layer_sums.append(xs.sum(0) if S else x)
    total = xs.sum(0) if S else x
    hn = rms_norm(total, w["final.norm"], eps)
    if rnd:
        hn = rnd(hn)
    return hn @ w["embed"].T, new_past


def round_to_bfloat16(t: torch.Tensor) -> torch.Tensor:
    """What an engine that stores activations in bfloat16 keeps of ``t`` (round to nearest even)."""
    return t.to(torch.bfloat16).to(t.dtype)
