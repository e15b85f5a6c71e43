"""Shared by the Zedudra tests: small configurations that differ in every size and option, random
weights by on-disk name (made here, not by the engine), and the plain model's logits."""
from __future__ import annotations

import copy
from typing import Dict, List, Optional

import numpy as np
import torch

from plain import zedudra_plain as plain


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(ff, limit, experts, top, groups=None, keep=None):
    router = {"experts": experts, "top": top}
    if groups is not None:
        router["groups"] = {"count": groups, "keep": keep}
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": router}


def attn(heads, kv_heads, dim, size, keep_first, rot_dims, base, scale, mlp, weights_of=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": dim, "scale": scale,
         "mask": {"size": size, "keep_first": keep_first}}
    if rot_dims:
        m["rot"] = {"dims": rot_dims, "base": base}
    layer = {"type": "attention", "mixer": m, "mlp": mlp}
    if weights_of is not None:
        layer["weights_of"] = weights_of
    return layer


def again(cfg_layers, j):
    """A layer that uses layer j's tensors: the rest of its entry equals layer j's."""
    layer = copy.deepcopy(cfg_layers[j])
    layer["weights_of"] = j
    return layer


def _with_shared(layers, shared):
    out = list(layers)
    for at, j in shared:
        out.insert(at, again(out, j))
    return out


# A: grouped heads, a window of 12 beside 5 kept positions (neither a multiple of the page), rotation over half a head,
# four norm groups, three taps; dense, routed (4 groups of 2, 2 kept, top 3), a layer run three times, a layer without feed-forward
ZED_A = {"architecture": "Zedudra", "vocab": 200, "width": 64, "norm": {"eps": 1e-5, "groups": 4}, "canon": {"taps": 3},
         "embedding": {"scale": 2.5},
         "layers": _with_shared([attn(4, 2, 16, 12, 5, 8, 10000.0, 0.3, dense(96)),
                                 attn(4, 2, 16, 12, 5, 8, 10000.0, 0.3, moe(24, 1.5, 8, 3, groups=4, keep=2)),
                                 attn(2, 1, 24, 20, 0, 24, 500.0, 0.2, None)], [(2, 1), (3, 1)])}
# B: nothing is a multiple of eight; every head its own keys, rotation over the whole head, no kept positions in one layer,
# five norm groups, two taps, a router without groups, a dense layer run twice
ZED_B = {"architecture": "Zedudra", "vocab": 77, "width": 50, "norm": {"eps": 3e-6, "groups": 5}, "canon": {"taps": 2},
         "embedding": {"scale": 0.7},
         "layers": _with_shared([attn(3, 3, 10, 7, 0, 10, 1000.0, 0.35, moe(22, 0.7, 6, 2)),
                                 attn(5, 1, 6, 9, 3, 2, 30.0, 0.4, dense(70))], [(2, 1)])}
# C: sizes that resemble a real model's heads (64 and 128), one norm group, four taps, kept positions that end inside a
# page and at a page's end, a window longer than a page run, groups of two experts (a group's worth is all it has)
ZED_C = {"architecture": "Zedudra", "vocab": 512, "width": 256, "norm": {"eps": 1e-6, "groups": 1}, "canon": {"taps": 4},
         "embedding": {"scale": 16.0},
         "layers": [attn(4, 1, 64, 40, 17, 32, 1000000.0, 0.125, dense(512)),
                    attn(2, 2, 128, 100, 64, 64, 40000.0, 0.09, moe(128, 2.0, 8, 2, groups=4, keep=2)),
                    attn(8, 2, 64, 33, 16, 64, 10000.0, 0.125, moe(64, 1.0, 4, 1, groups=2, keep=1))]}
# D: one head, one tap (no convolution state), no rotation, every expert chosen, more kept positions than the window is
# long, a window of one position (a query sees itself and the kept ones), as many norm groups as make pairs of columns
ZED_D = {"architecture": "Zedudra", "vocab": 90, "width": 32, "norm": {"eps": 1e-5, "groups": 16}, "canon": {"taps": 1},
         "embedding": {"scale": 1.0},
         "layers": [attn(1, 1, 12, 4, 30, 0, 1.0, 0.29, moe(16, 3.0, 3, 3, groups=1, keep=1)),
                    attn(1, 1, 20, 1, 6, 0, 1.0, 0.22, dense(40)),
                    attn(2, 2, 8, 1, 0, 4, 77.0, 0.35, None)]}
# E: no convolution at all (no state), a window longer than every request, groups of one expert, two norm groups
ZED_E = {"architecture": "Zedudra", "vocab": 120, "width": 48, "norm": {"eps": 1e-6, "groups": 2},
         "embedding": {"scale": 4.0},
         "layers": [attn(4, 4, 12, 5000, 3, 6, 9000.0, 0.3, moe(20, 1.2, 5, 2, groups=5, keep=3)),
                    attn(6, 2, 8, 31, 31, 8, 200.0, 0.35, dense(64))]}
ZED = {"A": ZED_A, "B": ZED_B, "C": ZED_C, "D": ZED_D, "E": ZED_E}


def owner(cfg: Dict, i: int) -> int:
    j = cfg["layers"][i].get("weights_of")
    return i if j is None else j


def tensor_shapes(cfg: Dict) -> Dict[str, tuple]:
    V, W = cfg["vocab"], cfg["width"]
    shapes = {"embed": (V, W), "head": (V, W), "final.norm": (W,)}
    taps = (cfg.get("canon") or {}).get("taps", 0)
    for i, layer in enumerate(cfg["layers"]):
        if layer.get("weights_of") is not None:
            continue
        p, m = f"l{i}.", layer["mixer"]
        H, G, D = m["heads"], m["kv_heads"], m["dim"]
        shapes.update({p + "norm1": (W,), p + "norm1b": (W,), p + "mix.q": (H * D, W), p + "mix.k": (G * D, W),
                       p + "mix.g": (H, W), p + "mix.o": (W, H * D)})
        if taps:
            shapes[p + "canon1"] = (W, taps)
        mlp = layer.get("mlp")
        if mlp is None:
            continue
        shapes.update({p + "norm2": (W,), p + "norm2b": (W,)})
        y = p + "mlp."
        if mlp["kind"] == "dense":
            shapes.update({y + "up": (mlp["ff"], W), y + "down": (W, mlp["ff"]), y + "act": (2,)})
        else:
            ff = mlp["expert"]["ff"]
            shapes[y + "router"] = (mlp["router"]["experts"], W)
            for e in range(mlp["router"]["experts"]):
                shapes.update({f"{y}e{e}.gate": (ff, W), f"{y}e{e}.up": (ff, W), f"{y}e{e}.down": (W, ff)})
    return shapes


def make_weights(cfg: Dict, seed: int, stored: torch.dtype = torch.bfloat16, router_gain: float = 3.0,
                 key_gain: float = 1.0) -> Dict[str, torch.Tensor]:
    """Matrices N(0, 1/sqrt(columns)), the embedding N(0, 1) / its scale; norm weights 1 + N(0, 0.1); convolution taps
    N(0, 0.5); the activation's two numbers N(0, 1). ``router_gain`` multiplies the router's matrix (spread scores, fewer
    near ties); ``key_gain`` the query and key matrices (steep softmax, so that a wrong key shows). Rounded to ``stored``."""
    g = torch.Generator().manual_seed(seed)
    out = {}
    for name, shape in tensor_shapes(cfg).items():
        if name.endswith("canon1"):
            t = 0.5 * torch.randn(shape, generator=g)
        elif name == "embed":
            t = torch.randn(shape, generator=g) / cfg["embedding"]["scale"]
        elif len(shape) == 2:
            t = torch.randn(shape, generator=g) / shape[1] ** 0.5
            if name.endswith(".router"):
                t = t * router_gain
            if name.endswith((".mix.q", ".mix.k")):
                t = t * key_gain
        elif name.endswith(".act"):
            t = torch.randn(shape, generator=g)
        else:
            t = 1.0 + 0.1 * torch.randn(shape, generator=g)
        out[name] = t.to(stored)
    return out


def as_f64(weights: Dict[str, torch.Tensor]) -> Dict[str, torch.Tensor]:
    return {k: v.to(torch.float64) for k, v in weights.items()}


def plain_logits(cfg: Dict, weights: Dict[str, torch.Tensor], tokens: List[int], rnd=None) -> np.ndarray:
    return plain.forward(cfg, as_f64(weights), tokens, rnd=rnd)[0].numpy()


def plain_logits_bf16(cfg: Dict, weights: Dict[str, torch.Tensor], tokens: List[int]) -> np.ndarray:
    return plain_logits(cfg, weights, tokens, rnd=plain.round_to_bfloat16)


def plain_logits_f32(cfg: Dict, weights: Dict[str, torch.Tensor], tokens: List[int]) -> np.ndarray:
    """The plain model evaluated in float32: how far 32-bit arithmetic alone moves the logits."""
    return plain.forward(cfg, {k: v.to(torch.float32) for k, v in weights.items()}, tokens)[0].numpy()


def random_tokens(cfg: Dict, n: int, seed: int) -> List[int]:
    rng = np.random.default_rng(seed)
    return [int(t) for t in rng.integers(0, cfg["vocab"], size=n)]


def with_layers(cfg: Dict, layers: List[Dict]) -> Dict:
    c = copy.deepcopy(cfg)
    c["layers"] = copy.deepcopy(layers)
    return c


def _divisors(n: int) -> List[int]:
    return [d for d in range(1, n + 1) if n % d == 0]


def random_config(rng, dense_only: bool = False) -> Dict:
    """A configuration drawn at random: width, norm groups, taps, two to six layers that each draw their own head
    counts, head size, window, kept positions, rotated channels and feed-forward, some of them second calls of an earlier
    layer. ``dense_only``: heads of 64 or 128 and no mixtures (bfloat16 then stays close to the plain model: no router's
    near tie can fall the other way)."""
    width = int(rng.choice([96, 128, 160, 192, 256, 320, 384]))
    groups = int(rng.choice([g for g in _divisors(width) if g <= 16]))
    owners, layers = [], []
    for i in range(int(rng.integers(2, 7))):
        if owners and rng.random() < 0.35:
            layers.append(again(layers, int(rng.choice(owners))))
            continue
        dim = int(rng.choice([64, 128] if dense_only else [16, 32, 48, 64, 96, 128]))
        heads = int(rng.choice([1, 2, 3, 4, 6, 8, 12]))
        rot = min(dim, int(rng.choice([0, 2, 8, 16, dim // 2, dim])))
        kind = rng.choice(["dense", "dense", "none"] if dense_only else ["dense", "moe", "moe", "none"])
        if kind == "dense":
            mlp = dense(int(rng.choice([64, 96, 200, 256, 512])))
        elif kind == "moe":
            E = int(rng.choice([4, 6, 8, 12, 16, 32]))
            g = int(rng.choice(_divisors(E)))
            keep = int(rng.integers(1, g + 1))
            mlp = moe(int(rng.choice([32, 64, 96, 128])), float(rng.choice([0.5, 1.0, 2.0, 7.0])), E,
                      int(rng.integers(1, min(8, E // g * keep) + 1)), groups=g, keep=keep)
        else:
            mlp = None
        owners.append(i)
        layers.append(attn(heads, int(rng.choice(_divisors(heads))), dim, int(rng.integers(1, 90)),
                           int(rng.choice([0, 1, 4, 16, 23, 33, 64])), rot - rot % 2, float(rng.choice([100.0, 10000.0, 1e6])),
                           float(rng.choice([dim ** -0.5, 0.11, 0.2])), mlp))
    return {"architecture": "Zedudra", "vocab": int(rng.integers(100, 1300)), "width": width,
            "norm": {"eps": float(rng.choice([1e-5, 1e-6])), "groups": groups}, "canon": {"taps": int(rng.integers(1, 6))},
            "embedding": {"scale": float(rng.choice([1.0, width ** 0.5]))}, "layers": layers}
