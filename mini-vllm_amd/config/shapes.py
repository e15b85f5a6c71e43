"""Named Qwen3 shapes for random-weights models: the sizes of the published Qwen3 dense models
(what their config.json files state) and a tiny one. Used by ``run.py --random-model`` and by the
benchmark; a shape is a dictionary of config.json keys that ``Qwen3Config.from_dict`` reads."""
from __future__ import annotations

from typing import Any, Dict

QWEN3_SHAPES: Dict[str, Dict[str, Any]] = {
    "tiny": dict(num_hidden_layers=2, hidden_size=64, num_attention_heads=4, num_key_value_heads=2, head_dim=16,
                 intermediate_size=128, vocab_size=256, rope_theta=10000.0, rms_norm_eps=1e-6,
                 tie_word_embeddings=True),
    "0.6b": dict(num_hidden_layers=28, hidden_size=1024, num_attention_heads=16, num_key_value_heads=8, head_dim=128,
                 intermediate_size=3072, vocab_size=151936, rope_theta=1e6, rms_norm_eps=1e-6,
                 tie_word_embeddings=True),
    "8b": dict(num_hidden_layers=36, hidden_size=4096, num_attention_heads=32, num_key_value_heads=8, head_dim=128,
               intermediate_size=12288, vocab_size=151936, rope_theta=1e6, rms_norm_eps=1e-6,
               tie_word_embeddings=False),
    "32b": dict(num_hidden_layers=64, hidden_size=5120, num_attention_heads=64, num_key_value_heads=8, head_dim=128,
                intermediate_size=25600, vocab_size=151936, rope_theta=1e6, rms_norm_eps=1e-6,
                tie_word_embeddings=False),
}


def named_shapes() -> Dict[str, Dict[str, Any]]:
    """Every named shape as a raw config.json dictionary, ``architectures`` included: the registry
    picks the architecture from it, as it does for a model folder. Another architecture's shapes are
    added here."""
    shapes = {name: qwen3_shape(name) for name in QWEN3_SHAPES}
    shapes["bolapel-tiny"] = bolapel_tiny_shape()
    shapes["dutilix-tiny"] = dutilix_tiny_shape()
    shapes["zedudra-tiny"] = zedudra_tiny_shape()
    shapes["furanex-tiny"] = furanex_tiny_shape()
    for name in QWEN3_SHAPES:
        if name != "tiny":
            shapes[f"bolapel-{name}"] = bolapel_shape(name)
            shapes[f"dutilix-{name}"] = dutilix_shape(name)
            shapes[f"zedudra-{name}"] = zedudra_shape(name)
            shapes[f"furanex-{name}"] = furanex_shape(name)
    return shapes


def named_shape(name: str, **overrides) -> Dict[str, Any]:
    shapes = named_shapes()
    if name not in shapes:
        raise KeyError(f"unknown shape {name!r} (known: {sorted(shapes)})")
    return dict(shapes[name], **overrides)


def qwen3_shape(name: str, **overrides) -> Dict[str, Any]:
    """The raw config dictionary of a named shape (``architectures`` and a position limit included)."""
    if name not in QWEN3_SHAPES:
        raise KeyError(f"unknown shape {name!r} (known: {sorted(QWEN3_SHAPES)})")
    raw = dict(QWEN3_SHAPES[name], architectures=["Qwen3ForCausalLM"], max_position_embeddings=40960)
    raw.update(overrides)
    return raw


def bolapel_shape(name: str, layers: int = None, chunk: int = 1024, delta_head_dim: int = 64, decay_rank: int = 64,
                  pattern: int = 4) -> Dict[str, Any]:
    """A Bolapel configuration with the width, feed-forward, vocabulary, head counts and head size of
    the named Qwen3 shape and as many layers: every ``pattern``-th layer is attention in chunks of
    ``chunk`` tokens (rotation over half of each head; every second of them reads the keys and values
    of the one before), the others are delta-rule layers with heads of ``delta_head_dim``. For
    random-weights models at sizes that resemble a real model's layers."""
    q = QWEN3_SHAPES[name]
    n = layers or q["num_hidden_layers"]
    hid, hd = q["hidden_size"], q["head_dim"]
    ff = {"kind": "dense", "ff": q["intermediate_size"]}
    out, owner = [], None
    for i in range(n):
        if i % pattern == pattern - 1:
            m = {"heads": q["num_attention_heads"], "kv_heads": q["num_key_value_heads"], "dim": hd, "vdim": hd,
                 "scale": hd ** -0.5, "mask": {"size": chunk}, "rot": {"dims": hd // 2, "base": q["rope_theta"]}}
            if owner is not None:
                m["kv_from"], owner = owner, None
            else:
                owner = i
            out.append({"type": "attention", "mixer": m, "mlp": ff})
        else:
            out.append({"type": "general_delta", "mlp": ff,
                        "mixer": {"heads": hid // delta_head_dim, "dim": delta_head_dim, "rank": decay_rank}})
    return {"architecture": "Bolapel", "vocab": q["vocab_size"], "width": hid, "layers": out,
            "norm": {"eps": q["rms_norm_eps"]}, "logit_softcap": 30.0}


def bolapel_tiny_shape() -> Dict[str, Any]:
    """A Bolapel model of a few thousand weights with every kind of layer: delta rule, attention in chunks
    with keys of its own, a layer without feed-forward, attention on another layer's keys."""
    ff = {"kind": "dense", "ff": 96}
    attn = {"heads": 4, "kv_heads": 2, "dim": 16, "vdim": 24, "scale": 0.25, "mask": {"size": 24},
            "rot": {"dims": 8, "base": 10000.0}}
    return {"architecture": "Bolapel", "vocab": 256, "width": 64, "norm": {"eps": 1e-5}, "logit_softcap": 20.0,
            "layers": [{"type": "general_delta", "mixer": {"heads": 2, "dim": 16, "rank": 8}, "mlp": ff},
                       {"type": "attention", "mixer": dict(attn), "mlp": ff},
                       {"type": "general_delta", "mixer": {"heads": 4, "dim": 8, "rank": 8}, "mlp": None},
                       {"type": "attention", "mixer": dict(attn, kv_from=1), "mlp": ff}]}


def dutilix_shape(name: str, layers: int = None, experts: int = 32, top: int = 4, identity: int = 0, groups: int = 4,
                  keep: int = 2, state_head_dim: int = 64, kv_rank: int = 256, rot_dim: int = 64, conv: int = 4,
                  pattern: int = 4) -> Dict[str, Any]:
    """A Dutilix configuration with the width, vocabulary, head count, head size and number of layers of the
    named Qwen3 shape: every ``pattern``-th layer is attention over a cached latent of ``kv_rank`` numbers (a
    rotated key part of ``rot_dim``), the others alternate between the gated delta rule (a query/key group for
    every two heads) and the mLSTM, both with heads of ``state_head_dim``. Every second feed-forward is a mixture
    of ``experts`` experts of which ``top`` are used, each 1/top of the shape's dense width, the others are dense.
    For random-weights models at sizes that resemble a real model's layers."""
    q = QWEN3_SHAPES[name]
    n = layers or q["num_hidden_layers"]
    hid, hd, heads = q["hidden_size"], q["head_dim"], q["num_attention_heads"]
    state_heads = hid // state_head_dim
    dense = {"kind": "dense", "ff": q["intermediate_size"]}
    sparse = {"kind": "moe", "expert": {"ff": q["intermediate_size"] // top},
              "router": {"experts": experts, "identity": identity, "top": top, "groups": {"count": groups, "keep": keep}}}
    out = []
    for i in range(n):
        mlp = sparse if i % 2 else dense
        if i % pattern == pattern - 1:
            m = {"heads": heads, "dim": hd, "rot_dim": rot_dim, "vdim": hd, "q_rank": max(64, hid // 4), "kv_rank": kv_rank,
                 "scale": (hd + rot_dim) ** -0.5, "rot": {"dims": rot_dim, "base": q["rope_theta"]}}
            out.append({"type": "latent_attention", "mixer": m, "mlp": mlp})
        elif i % 2 == 0:
            out.append({"type": "delta", "mlp": mlp, "mixer": {"heads": state_heads, "kv_heads": max(1, state_heads // 2),
                                                               "dim": state_head_dim, "vdim": state_head_dim, "conv": conv}})
        else:
            out.append({"type": "mlstm", "mlp": mlp, "mixer": {"heads": state_heads, "dim": state_head_dim,
                                                               "vdim": state_head_dim, "gate_cap": 15.0}})
    return {"architecture": "Dutilix", "vocab": q["vocab_size"], "width": hid, "layers": out,
            "norm": {"eps": q["rms_norm_eps"]}, "logit_scale": 1.0}


def dutilix_tiny_shape() -> Dict[str, Any]:
    """A Dutilix model of a few thousand weights with every kind of layer and feed-forward."""
    moe = {"kind": "moe", "expert": {"ff": 32},
           "router": {"experts": 6, "identity": 2, "top": 2, "groups": {"count": 4, "keep": 2}}}
    return {"architecture": "Dutilix", "vocab": 256, "width": 64, "norm": {"eps": 1e-5}, "logit_scale": 0.5,
            "layers": [{"type": "delta", "mixer": {"heads": 4, "kv_heads": 2, "dim": 8, "vdim": 16, "conv": 3}, "mlp": moe},
                       {"type": "latent_attention", "mlp": {"kind": "dense", "ff": 96},
                        "mixer": {"heads": 4, "dim": 12, "rot_dim": 4, "vdim": 8, "q_rank": 24, "kv_rank": 16, "scale": 0.25,
                                  "rot": {"dims": 4, "base": 10000.0}}},
                       {"type": "mlstm", "mixer": {"heads": 2, "dim": 16, "vdim": 24, "gate_cap": 12.0}, "mlp": None}]}


def zedudra_shape(name: str, layers: int = None, window: int = 1024, keep_first: int = 64, experts: int = 32, top: int = 4,
                  groups: int = 4, keep: int = 2, taps: int = 4, norm_groups: int = 4, limit: float = 7.0,
                  dense_every: int = 2) -> Dict[str, Any]:
    """A Zedudra configuration with the width, vocabulary, head counts, head size and number of layers of the named
    Qwen3 shape: every layer is attention over a window of ``window`` positions beside the first ``keep_first``, with a
    rotation over half of each head; every ``dense_every``-th feed-forward (from the first) is dense at the shape's
    width, the others are mixtures of ``experts`` experts of which ``top`` are used, each 1/top of the dense width.
    For random-weights models at sizes that resemble a real model's layers."""
    q = QWEN3_SHAPES[name]
    n = layers or q["num_hidden_layers"]
    hid, hd = q["hidden_size"], q["head_dim"]
    dense = {"kind": "dense", "ff": q["intermediate_size"]}
    sparse = {"kind": "moe", "expert": {"ff": q["intermediate_size"] // top, "limit": limit},
              "router": {"experts": experts, "top": top, "groups": {"count": groups, "keep": keep}}}
    mixer = {"heads": q["num_attention_heads"], "kv_heads": q["num_key_value_heads"], "dim": hd, "vdim": hd,
             "scale": hd ** -0.5, "mask": {"size": window, "keep_first": keep_first},
             "rot": {"dims": hd // 2, "base": q["rope_theta"]}}
    out = [{"type": "attention", "mixer": dict(mixer), "mlp": dense if i % dense_every == 0 else sparse} for i in range(n)]
    return {"architecture": "Zedudra", "vocab": q["vocab_size"], "width": hid, "layers": out,
            "norm": {"eps": q["rms_norm_eps"], "groups": norm_groups}, "canon": {"taps": taps},
            "embedding": {"scale": float(hid) ** 0.5}}


def zedudra_tiny_shape() -> Dict[str, Any]:
    """A Zedudra model of a few thousand weights: a dense layer, a routed layer that runs twice, a layer without
    feed-forward."""
    mixer = {"heads": 4, "kv_heads": 2, "dim": 16, "vdim": 16, "scale": 0.25, "mask": {"size": 24, "keep_first": 4},
             "rot": {"dims": 8, "base": 10000.0}}
    moe = {"kind": "moe", "expert": {"ff": 32, "limit": 2.0}, "router": {"experts": 8, "top": 2, "groups": {"count": 4, "keep": 2}}}
    return {"architecture": "Zedudra", "vocab": 256, "width": 64, "norm": {"eps": 1e-5, "groups": 2}, "canon": {"taps": 3},
            "embedding": {"scale": 8.0},
            "layers": [{"type": "attention", "mixer": dict(mixer), "mlp": {"kind": "dense", "ff": 96}},
                       {"type": "attention", "mixer": dict(mixer), "mlp": moe},
                       {"type": "attention", "mixer": dict(mixer), "mlp": moe, "weights_of": 1},
                       {"type": "attention", "mixer": dict(mixer, kv_heads=4), "mlp": None}]}


def furanex_shape(name: str, layers: int = None, streams: int = 4, experts: int = 32, top: int = 4, shared: bool = True,
                  latent_every: int = 2) -> Dict[str, Any]:
    """A Furanex configuration with the width, vocabulary, head counts, head size and number of layers of the named Qwen3
    shape: every ``latent_every``-th layer (from the second) is attention over a latent of 256 with 64 rotated channels
    and a query latent of a quarter of the width, the others are grouped attention whose values are shared along the
    layers; every feed-forward is a mixture of ``experts`` experts of which ``top`` are used, each 1/top of the shape's
    dense width, beside a shared expert of the same size. For random-weights models at sizes that resemble a real
    model's layers."""
    q = QWEN3_SHAPES[name]
    n = layers or q["num_hidden_layers"]
    hid, hd = q["hidden_size"], q["head_dim"]
    stretch = {"factor": 8.0, "original": 4096, "fast": 32.0, "slow": 1.0}
    attention = {"heads": q["num_attention_heads"], "kv_heads": q["num_key_value_heads"], "dim": hd, "vdim": hd,
                 "scale": 8.0 / hd, "v_mix": True, "rot": {"dims": hd, "base": q["rope_theta"], "scaling": dict(stretch)}}
    latent = {"heads": q["num_attention_heads"], "dim": hd, "rot_dim": 64, "vdim": hd, "q_rank": max(64, hid // 4),
              "kv_rank": 256, "scale": (hd + 64) ** -0.5, "rot": {"dims": 64, "base": 10000.0, "scaling": dict(stretch)}}
    mlp = {"kind": "moe", "expert": {"ff": q["intermediate_size"] // top}, "router": {"experts": experts, "top": top}}
    if shared:
        mlp["shared"] = {"ff": q["intermediate_size"] // top}
    out = [{"type": "latent_attention" if i % latent_every == latent_every - 1 else "attention",
            "mixer": dict(latent if i % latent_every == latent_every - 1 else attention), "mlp": dict(mlp)} for i in range(n)]
    return {"architecture": "Furanex", "vocab": q["vocab_size"], "width": hid, "streams": streams, "layers": out,
            "norm": {"eps": q["rms_norm_eps"]}, "embedding": {"scale": float(hid) ** 0.5}}


def furanex_tiny_shape() -> Dict[str, Any]:
    """A Furanex model of a few thousand weights: two value-sharing attention layers around a latent-attention layer,
    one of them without a feed-forward."""
    stretch = {"factor": 3.0, "original": 64, "fast": 16.0, "slow": 2.0}
    attention = {"heads": 4, "kv_heads": 2, "dim": 16, "vdim": 8, "scale": 0.2, "v_mix": True,
                 "rot": {"dims": 12, "base": 5000.0, "scaling": dict(stretch)}}
    latent = {"heads": 3, "dim": 12, "rot_dim": 4, "vdim": 8, "q_rank": 24, "kv_rank": 16, "scale": 0.25,
              "rot": {"dims": 4, "base": 10000.0, "scaling": dict(stretch)}}
    moe = {"kind": "moe", "expert": {"ff": 24}, "router": {"experts": 5, "top": 2}, "shared": {"ff": 40}}
    return {"architecture": "Furanex", "vocab": 256, "width": 48, "streams": 3, "norm": {"eps": 1e-5}, "embedding": {"scale": 6.0},
            "layers": [{"type": "attention", "mixer": dict(attention), "mlp": dict(moe)},
                       {"type": "latent_attention", "mixer": dict(latent), "mlp": None},
                       {"type": "attention", "mixer": dict(attention), "mlp": dict(moe)}]}
