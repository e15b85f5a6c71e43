"""Shared by the Furanex tests: small configurations that differ in every size and option, random
weights by on-disk name (made here, not by the engine), and the plain model's logits."""
from __future__ import annotations

import copy
from typing import Dict, List, Optional

import numpy as np
import torch

from plain import furanex_plain as plain


def stretch(factor, original, fast, slow):
    return {"factor": factor, "original": original, "fast": fast, "slow": slow}


def moe(ff, experts, top, shared=None):
    d = {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}
    if shared:
        d["shared"] = {"ff": shared}
    return d


def attn(heads, kv_heads, dim, vdim, rot_dims, base, scale, mlp, v_mix=True, scaling=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale, "v_mix": v_mix}
    if rot_dims:
        m["rot"] = {"dims": rot_dims, "base": base}
        if scaling:
            m["rot"]["scaling"] = scaling
    return {"type": "attention", "mixer": m, "mlp": mlp}


def latent(heads, dim, rot_dim, vdim, q_rank, kv_rank, base, scale, mlp, scaling=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank, "scale": scale}
    if rot_dim:
        m["rot"] = {"dims": rot_dim, "base": base}
        if scaling:
            m["rot"]["scaling"] = scaling
    return {"type": "latent_attention", "mixer": m, "mlp": mlp}


# A: three streams; grouped heads with values smaller than keys, rotation over part of a head with stretched
# frequencies whose ramp lies inside the pairs; a latent layer without a feed-forward between two value-sharing layers;
# two experts a token beside a shared expert of another width
FUR_A = {"architecture": "Furanex", "vocab": 200, "width": 48, "streams": 3, "norm": {"eps": 1e-5}, "embedding": {"scale": 6.0},
         "layers": [attn(4, 2, 16, 8, 12, 5000.0, 0.2, moe(24, 5, 2, shared=40), scaling=stretch(3.0, 64, 16.0, 2.0)),
                    latent(3, 12, 4, 8, 24, 16, 10000.0, 0.25, None, scaling=stretch(2.0, 32, 8.0, 1.0)),
                    attn(4, 2, 16, 8, 12, 5000.0, 0.2, moe(24, 5, 2, shared=40), scaling=stretch(3.0, 64, 16.0, 2.0))]}
# B: nothing is a multiple of eight; two streams; the latent layer first; every head its own keys; values larger than
# keys; one attention layer that shares no values between two that do; no shared expert; one expert a token; plain
# frequencies in one layer, rotation over the whole head
FUR_B = {"architecture": "Furanex", "vocab": 77, "width": 50, "streams": 2, "norm": {"eps": 3e-6}, "embedding": {"scale": 0.7},
         "layers": [latent(5, 6, 2, 10, 14, 18, 300.0, 0.3, moe(22, 3, 1)),
                    attn(3, 3, 10, 14, 10, 1000.0, 0.35, moe(18, 6, 3), scaling=stretch(8.0, 16, 4.0, 0.5)),
                    attn(2, 1, 6, 4, 2, 30.0, 0.4, None, v_mix=False),
                    attn(6, 3, 12, 14, 6, 77.0, 0.3, moe(10, 4, 4, shared=26))]}
# C: sizes that resemble a real model's heads (64 and 128, latents of 128 and 256 with 32 and 64 rotated channels),
# four streams, as the MFMA and vector kernels take them
FUR_C = {"architecture": "Furanex", "vocab": 512, "width": 256, "streams": 4, "norm": {"eps": 1e-6}, "embedding": {"scale": 16.0},
         "layers": [attn(6, 2, 64, 64, 64, 500000.0, 0.1, moe(96, 10, 2, shared=64), scaling=stretch(8.0, 2048, 16.0, 2.0)),
                    latent(8, 64, 32, 32, 96, 128, 20000.0, 0.1, moe(96, 10, 2, shared=64), scaling=stretch(4.0, 256, 16.0, 1.0)),
                    attn(6, 2, 64, 64, 64, 500000.0, 0.1, moe(128, 8, 1, shared=32), scaling=stretch(8.0, 2048, 16.0, 2.0)),
                    latent(16, 64, 64, 64, 96, 256, 50000.0, 0.09, moe(32, 4, 2)),
                    attn(2, 1, 128, 128, 128, 10000.0, 0.09, None, v_mix=False)]}
# D: one stream, one head everywhere, no rotation at all in one layer and no rotated part in the latent layer, every
# expert chosen, a single value-sharing layer (nothing to blend with)
FUR_D = {"architecture": "Furanex", "vocab": 90, "width": 32, "streams": 1, "norm": {"eps": 1e-5}, "embedding": {"scale": 1.0},
         "layers": [attn(1, 1, 12, 12, 0, 1.0, 0.29, moe(16, 3, 3, shared=8)),
                    latent(1, 20, 0, 6, 10, 12, 1.0, 0.22, moe(12, 2, 1)),
                    attn(2, 2, 8, 20, 4, 77.0, 0.35, None, v_mix=False)]}
# E: no streams named (one plain residual), attention layers only, a stretch factor whose ramp covers every pair
FUR_E = {"architecture": "Furanex", "vocab": 120, "width": 40, "norm": {"eps": 1e-6}, "embedding": {"scale": 4.0},
         "layers": [attn(4, 4, 12, 10, 12, 9000.0, 0.3, moe(20, 5, 2), scaling=stretch(2.0, 4000, 1000.0, 0.001)),
                    attn(8, 4, 8, 10, 8, 200.0, 0.35, moe(16, 7, 3, shared=12))]}
FUR = {"A": FUR_A, "B": FUR_B, "C": FUR_C, "D": FUR_D, "E": FUR_E}


def tensor_shapes(cfg: Dict) -> Dict[str, tuple]:
    V, W, S = cfg["vocab"], cfg["width"], cfg.get("streams")
    shapes = {"embed": (V, W), "final.norm": (W,)}
    for i, layer in enumerate(cfg["layers"]):
        p, m = f"l{i}.", layer["mixer"]
        shapes[p + "norm1"] = (W,)
        if S:
            shapes.update({p + "hc1.in": (S,), p + "hc1.out": (S,), p + "hc1.mix": (S, S)})
        x = p + "mix."
        if layer["type"] == "attention":
            H, G, D, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
            shapes.update({x + "q": (H * D, W), x + "k": (G * D, W), x + "v": (G * Dv, W), x + "o": (W, H * Dv)})
            if m.get("v_mix"):
                shapes[x + "vmix"] = ()
        else:
            H, D, Dr, Dv, Q, R = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["q_rank"], m["kv_rank"]
            shapes.update({x + "dq": (Q, W), x + "dq.norm": (Q,), x + "uq": (H * (D + Dr), Q), x + "dkv": (R + Dr, W),
                           x + "dkv.norm": (R,), x + "uk": (H * D, R), x + "uv": (H * Dv, R), x + "g": (H, W), x + "o": (W, H * Dv)})
        mlp = layer.get("mlp")
        if mlp is None:
            continue
        shapes[p + "norm2"] = (W,)
        if S:
            shapes.update({p + "hc2.in": (S,), p + "hc2.out": (S,), p + "hc2.mix": (S, S)})
        y, ff = p + "mlp.", mlp["expert"]["ff"]
        shapes[y + "table"] = (V, mlp["router"]["top"])
        for e in range(mlp["router"]["experts"]):
            shapes.update({f"{y}e{e}.gate": (ff, W), f"{y}e{e}.up": (ff, W), f"{y}e{e}.down": (W, ff)})
        if mlp.get("shared"):
            fs = mlp["shared"]["ff"]
            shapes.update({y + "shared.gate": (fs, W), y + "shared.up": (fs, W), y + "shared.down": (W, fs)})
    return shapes


def make_weights(cfg: Dict, seed: int, stored: torch.dtype = torch.bfloat16, key_gain: float = 1.0) -> Dict[str, torch.Tensor]:
    """Matrices N(0, 1/sqrt(columns)), the embedding N(0, 1) / its scale; norm weights 1 + N(0, 0.1); stream weights: reads
    1/S + N(0, 0.1), writes 1 + N(0, 0.2), the mixing matrix the identity + N(0, 0.15); the blend weight of shared values
    in (0.2, 0.8); tables: rows of distinct experts. ``key_gain`` multiplies the attention's scale through the query
    matrix of the latent layers and is applied to ``scale`` by the caller for the others (q and k are unit vectors there).
    Rounded to ``stored``; integer tables are int32."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    S = cfg.get("streams") or 1
    for name, shape in tensor_shapes(cfg).items():
        if name.endswith(".table"):
            layer = cfg["layers"][int(name.split(".")[0][1:])]
            E = layer["mlp"]["router"]["experts"]
            out[name] = torch.rand((shape[0], E), generator=g).argsort(dim=1)[:, :shape[1]].to(torch.int32).contiguous()
            continue
        if name == "embed":
            t = torch.randn(shape, generator=g) / cfg["embedding"]["scale"]
        elif name.endswith(".vmix"):
            t = 0.2 + 0.6 * torch.rand(shape, generator=g)
        elif ".hc" in name and name.endswith(".in"):
            t = 1.0 / S + 0.1 * torch.randn(shape, generator=g)
        elif ".hc" in name and name.endswith(".out"):
            t = 1.0 + 0.2 * torch.randn(shape, generator=g)
        elif ".hc" in name and name.endswith(".mix"):
            t = torch.eye(S) + 0.15 * torch.randn(shape, generator=g)
        elif len(shape) == 2:
            t = torch.randn(shape, generator=g) / shape[1] ** 0.5
            if name.endswith(".mix.uq"):
                t = t * key_gain
        else:
            t = 1.0 + 0.1 * torch.randn(shape, generator=g)
        out[name] = t.to(stored)
    return out


def sharpened(cfg: Dict, gain: float) -> Dict:
    """The configuration with the scale of every grouped-attention layer multiplied: its q and k are unit vectors, so a
    steeper softmax (one lost key shows) comes from the scale alone."""
    c = copy.deepcopy(cfg)
    for layer in c["layers"]:
        if layer["type"] == "attention":
            layer["mixer"]["scale"] *= gain
    return c


def as_f64(weights: Dict[str, torch.Tensor]) -> Dict[str, torch.Tensor]:
    return {k: (v.to(torch.float64) if v.is_floating_point() else v) for k, v in weights.items()}


def plain_logits(cfg: Dict, weights: Dict[str, torch.Tensor], tokens: List[int], rnd=None) -> np.ndarray:
    return plain.forward(cfg, as_f64(weights), tokens, rnd=rnd)[0].numpy()


def plain_logits_bf16(cfg: Dict, weights: Dict[str, torch.Tensor], tokens: List[int]) -> np.ndarray:
    return plain_logits(cfg, weights, tokens, rnd=plain.round_to_bfloat16)


def plain_logits_f32(cfg: Dict, weights: Dict[str, torch.Tensor], tokens: List[int]) -> np.ndarray:
    """The plain model evaluated in float32: how far 32-bit arithmetic alone moves the logits."""
    w = {k: (v.to(torch.float32) if v.is_floating_point() else v) for k, v in weights.items()}
    return plain.forward(cfg, w, tokens)[0].numpy()


def random_tokens(cfg: Dict, n: int, seed: int) -> List[int]:
    rng = np.random.default_rng(seed)
    return [int(t) for t in rng.integers(0, cfg["vocab"], size=n)]


def _divisors(n: int) -> List[int]:
    return [d for d in range(1, n + 1) if n % d == 0]


def random_config(rng, fast_sizes: bool = False) -> Dict:
    """A configuration drawn at random: width, streams, two to six layers of either kind in any order, each drawing its
    own head counts, sizes, rotated channels, stretch and feed-forward; the value-sharing layers agree in kv heads and
    value size, as they must. ``fast_sizes``: heads of 64 or 128 and latents the MFMA kernels take."""
    width = int(rng.choice([96, 128, 160, 192, 256, 320]))
    shared_kv, shared_vdim = int(rng.choice([1, 2, 4])), int(rng.choice([64, 128] if fast_sizes else [8, 24, 40, 64]))
    layers = []
    for _ in range(int(rng.integers(2, 7))):
        E = int(rng.choice([2, 3, 5, 8, 12, 16]))
        kind = rng.choice(["moe", "moe", "shared", "none"])
        mlp = None if kind == "none" else moe(int(rng.choice([32, 64, 96])), E, int(rng.integers(1, min(4, E) + 1)),
                                              shared=int(rng.choice([16, 64, 96])) if kind == "shared" else None)
        sc = None if rng.random() < 0.3 else stretch(float(rng.choice([2.0, 4.0, 8.0])), int(rng.choice([32, 256, 1024])),
                                                       float(rng.choice([8.0, 32.0])), float(rng.choice([0.5, 1.0, 2.0])))
        base = float(rng.choice([100.0, 10000.0, 1e6]))
        if rng.random() < 0.6:
            dim = int(rng.choice([64, 128] if fast_sizes else [16, 24, 48, 64, 96]))
            share = rng.random() < 0.7
            kv = shared_kv if share else int(rng.choice([1, 2, 3]))
            heads = kv * int(rng.choice([1, 2, 4]))
            vdim = shared_vdim if share else (dim if fast_sizes else int(rng.choice([8, 16, dim])))
            if fast_sizes and share:
                dim = vdim
            rot = dim if fast_sizes else int(rng.choice([0, 2, dim // 2 - dim // 2 % 2, dim]))
            # (q and k are unit vectors: a score is at most scale * dim)
            layers.append(attn(heads, kv, dim, vdim, rot, base, float(rng.choice([4.0, 8.0, 12.0])) / dim, mlp, v_mix=share, scaling=sc))
        else:
            R, Dr = (int(x) for x in (rng.choice([(64, 32), (128, 32), (128, 64), (256, 64)]) if fast_sizes
                                      else rng.choice([(16, 4), (24, 0), (40, 8), (64, 16)])))
            layers.append(latent(int(rng.choice([1, 2, 4, 6])), int(rng.choice([32, 64] if fast_sizes else [8, 12, 32])), Dr,
                                 int(rng.choice([32, 64] if fast_sizes else [8, 20, 32])), int(rng.choice([32, 48, 96])), R, base,
                                 float(rng.choice([0.1, 0.2])), mlp, scaling=sc if Dr else None))
    cfg = {"architecture": "Furanex", "vocab": int(rng.integers(100, 1300)), "width": width,
           "norm": {"eps": float(rng.choice([1e-5, 1e-6]))}, "embedding": {"scale": float(rng.choice([1.0, width ** 0.5]))},
           "layers": layers}
    streams = int(rng.choice([0, 1, 2, 3, 4, 5]))
    if streams:
        cfg["streams"] = streams
    return cfg
