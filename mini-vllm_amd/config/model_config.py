"""Typed model configurations read from a model folder's ``config.json``.

Every size and constant of a model comes from here; no part of the engine carries a
default of its own for something ``config.json`` states.

Reference: the reference hands the raw ``transformers`` config object to the model
(minivllm/config/config.py:50, minivllm/models/loader.py:14) and the model reads
``head_dim``, ``num_attention_heads``, ``num_key_value_heads``, ``hidden_size``,
``intermediate_size``, ``rms_norm_eps``, ``rope_theta``, ``max_position_embeddings``,
``attention_bias``, ``tie_word_embeddings``, ``vocab_size``, ``num_hidden_layers``
(minivllm/models/models/qwen3.py:28-65,160-204). Here the same keys are parsed with
plain ``json`` into a frozen dataclass and validated.
"""
from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import Any, ClassVar, Dict, Optional, Tuple


class ConfigError(ValueError):
    """A ``config.json`` that the engine cannot serve correctly."""


_DTYPE_NAMES = {
    "bfloat16": "bfloat16", "bf16": "bfloat16", "torch.bfloat16": "bfloat16",
    "float32": "float32", "fp32": "float32", "float": "float32", "torch.float32": "float32",
    "float16": "float16", "fp16": "float16", "half": "float16", "torch.float16": "float16",
}


def _require(d: Dict[str, Any], key: str, typ, where: str):
    if key not in d or d[key] is None:
        raise ConfigError(f"{where}: required key '{key}' is missing")
    return _typed(d[key], key, typ, where)


def _typed(v, key: str, typ, where: str):
    if typ is int:
        if isinstance(v, bool) or not isinstance(v, int):
            raise ConfigError(f"{where}: key '{key}' must be an integer, got {v!r}")
        return v
    if typ is float:
        if isinstance(v, bool) or not isinstance(v, (int, float)):
            raise ConfigError(f"{where}: key '{key}' must be a number, got {v!r}")
        return float(v)
    if typ is bool:
        if not isinstance(v, bool):
            raise ConfigError(f"{where}: key '{key}' must be true or false, got {v!r}")
        return v
    raise TypeError(typ)


@dataclass(frozen=True)
class ModelConfig:
    """Base of all architecture configurations.

    A subclass names the ``architectures[0]`` string it serves in ``architecture`` and
    parses its own keys in ``from_dict``; ``to_dict`` writes them back under the same
    names so that a configuration can be stored as a ``config.json`` again.
    """

    architecture: ClassVar[str] = ""

    @classmethod
    def from_dict(cls, d: Dict[str, Any], where: str = "config.json") -> "ModelConfig":
        raise NotImplementedError

    def to_dict(self) -> Dict[str, Any]:
        raise NotImplementedError


@dataclass(frozen=True)
class Qwen3Config(ModelConfig):
    """Qwen3 dense decoder (reference: minivllm/models/models/qwen3.py).

    The reference's Qwen3 never passes a window to its attention layer (qwen3.py:66-71), so
    there every layer sees all keys whatever ``use_sliding_window`` says. Here the key is
    honoured with the meaning it has where it comes from: with ``use_sliding_window`` the
    layers with index >= ``max_window_layers`` see ``sliding_window`` keys, the query's own
    among them (key position > query position - sliding_window); the other layers see all.
    No file of the reference pins this: parity unpinned. The attention part counts a window as
    tokens to the left of the query besides itself (the reference's attention layer,
    minivllm/models/layers/attention.py:56-60), which is ``sliding_window - 1``.
    """

    architecture: ClassVar[str] = "Qwen3ForCausalLM"

    vocab_size: int = 0
    hidden_size: int = 0
    num_hidden_layers: int = 0
    num_attention_heads: int = 0
    num_key_value_heads: int = 0
    head_dim: int = 0
    intermediate_size: int = 0
    max_position_embeddings: int = 0
    rms_norm_eps: float = 1e-6
    rope_theta: float = 10000.0
    attention_bias: bool = False
    tie_word_embeddings: bool = False
    use_sliding_window: bool = False
    sliding_window: Optional[int] = None
    max_window_layers: int = 0
    dtype: str = "bfloat16"
    eos_token_ids: Tuple[int, ...] = ()
    bos_token_id: Optional[int] = None

    @property
    def q_dim(self) -> int:
        return self.num_attention_heads * self.head_dim

    @property
    def kv_dim(self) -> int:
        return self.num_key_value_heads * self.head_dim

    def layer_window(self, layer: int) -> Optional[int]:
        """How many tokens to the left of a query ``layer`` sees besides the query itself
        (``sliding_window`` keys in all, the query's own included), or None for all."""
        if self.use_sliding_window and layer >= self.max_window_layers:
            return self.sliding_window - 1
        return None

    @classmethod
    def from_dict(cls, d: Dict[str, Any], where: str = "config.json") -> "Qwen3Config":
        hidden = _require(d, "hidden_size", int, where)
        heads = _require(d, "num_attention_heads", int, where)
        kv_heads = d.get("num_key_value_heads")
        kv_heads = heads if kv_heads is None else _typed(kv_heads, "num_key_value_heads", int, where)
        head_dim = d.get("head_dim")
        if head_dim is None:
            # the reference's cache sizing falls back the same way (minivllm/executor/executor.py:41)
            if hidden % heads:
                raise ConfigError(f"{where}: no 'head_dim' and hidden_size {hidden} is not divisible by "
                                  f"num_attention_heads {heads}")
            head_dim = hidden // heads
        else:
            head_dim = _typed(head_dim, "head_dim", int, where)

        act = d.get("hidden_act", "silu")
        if act != "silu":
            # the reference applies SiLU whatever the key says (minivllm/models/models/qwen3.py:119)
            raise ConfigError(f"{where}: hidden_act '{act}' is not supported; Qwen3's feed-forward uses 'silu'")
        scaling = d.get("rope_scaling")
        if scaling not in (None, {}):
            rtype = scaling.get("rope_type", scaling.get("type")) if isinstance(scaling, dict) else scaling
            if rtype not in (None, "default"):
                raise ConfigError(f"{where}: rope_scaling {scaling!r} is not supported (plain rotary "
                                  f"embedding with rope_theta only)")
        if "rope_parameters" in d and isinstance(d["rope_parameters"], dict):
            rp = d["rope_parameters"]
            if rp.get("rope_type", "default") != "default":
                raise ConfigError(f"{where}: rope_parameters {rp!r} is not supported")
            if "rope_theta" not in d and "rope_theta" in rp:
                d = dict(d, rope_theta=rp["rope_theta"])

        use_window = d.get("use_sliding_window", False)
        use_window = False if use_window is None else _typed(use_window, "use_sliding_window", bool, where)
        window = d.get("sliding_window")
        layers = _require(d, "num_hidden_layers", int, where)
        max_window_layers = d.get("max_window_layers")
        if use_window:
            if window is None:
                raise ConfigError(f"{where}: use_sliding_window is true but 'sliding_window' is missing")
            window = _typed(window, "sliding_window", int, where)
            if window < 1:
                raise ConfigError(f"{where}: sliding_window counts the keys a query sees, its own included, "
                                  f"and must be >= 1, got {window}")
            max_window_layers = layers if max_window_layers is None else _typed(
                max_window_layers, "max_window_layers", int, where)
        else:
            window = None if window is None else _typed(window, "sliding_window", int, where)
            max_window_layers = layers if max_window_layers is None else _typed(
                max_window_layers, "max_window_layers", int, where)

        dtype = d.get("dtype", d.get("torch_dtype", "bfloat16"))
        if dtype is None:
            dtype = "bfloat16"
        if str(dtype) not in _DTYPE_NAMES:
            raise ConfigError(f"{where}: unknown dtype {dtype!r}")
        dtype = _DTYPE_NAMES[str(dtype)]

        eos = d.get("eos_token_id")
        if eos is None:
            eos_ids: Tuple[int, ...] = ()
        elif isinstance(eos, int) and not isinstance(eos, bool):
            eos_ids = (eos,)
        elif isinstance(eos, (list, tuple)) and all(isinstance(e, int) for e in eos):
            eos_ids = tuple(eos)
        else:
            raise ConfigError(f"{where}: eos_token_id must be an integer or a list of integers, got {eos!r}")
        bos = d.get("bos_token_id")

        cfg = cls(
            vocab_size=_require(d, "vocab_size", int, where),
            hidden_size=hidden,
            num_hidden_layers=layers,
            num_attention_heads=heads,
            num_key_value_heads=kv_heads,
            head_dim=head_dim,
            intermediate_size=_require(d, "intermediate_size", int, where),
            max_position_embeddings=_require(d, "max_position_embeddings", int, where),
            rms_norm_eps=_typed(d.get("rms_norm_eps", 1e-6), "rms_norm_eps", float, where),
            rope_theta=_typed(d.get("rope_theta", 10000.0), "rope_theta", float, where),
            attention_bias=_typed(d.get("attention_bias", False) or False, "attention_bias", bool, where),
            tie_word_embeddings=_typed(d.get("tie_word_embeddings", False) or False,
                                       "tie_word_embeddings", bool, where),
            use_sliding_window=use_window,
            sliding_window=window,
            max_window_layers=max_window_layers,
            dtype=dtype,
            eos_token_ids=eos_ids,
            bos_token_id=bos if isinstance(bos, int) else None,
        )
        cfg.validate(where)
        return cfg

    def validate(self, where: str = "config") -> None:
        for name in ("vocab_size", "hidden_size", "num_hidden_layers", "num_attention_heads",
                     "num_key_value_heads", "head_dim", "intermediate_size", "max_position_embeddings"):
            if getattr(self, name) <= 0:
                raise ConfigError(f"{where}: {name} must be positive, got {getattr(self, name)}")
        if self.num_attention_heads % self.num_key_value_heads:
            raise ConfigError(f"{where}: num_attention_heads {self.num_attention_heads} is not a multiple of "
                              f"num_key_value_heads {self.num_key_value_heads}")
        if self.head_dim % 2:
            raise ConfigError(f"{where}: head_dim {self.head_dim} must be even for the rotary embedding")
        if self.rms_norm_eps <= 0:
            raise ConfigError(f"{where}: rms_norm_eps must be positive, got {self.rms_norm_eps}")
        if self.rope_theta <= 0:
            raise ConfigError(f"{where}: rope_theta must be positive, got {self.rope_theta}")

    def to_dict(self) -> Dict[str, Any]:
        eos: Any
        if len(self.eos_token_ids) == 0:
            eos = None
        elif len(self.eos_token_ids) == 1:
            eos = self.eos_token_ids[0]
        else:
            eos = list(self.eos_token_ids)
        return {
            "architectures": [self.architecture],
            "model_type": "qwen3",
            "vocab_size": self.vocab_size,
            "hidden_size": self.hidden_size,
            "num_hidden_layers": self.num_hidden_layers,
            "num_attention_heads": self.num_attention_heads,
            "num_key_value_heads": self.num_key_value_heads,
            "head_dim": self.head_dim,
            "intermediate_size": self.intermediate_size,
            "max_position_embeddings": self.max_position_embeddings,
            "rms_norm_eps": self.rms_norm_eps,
            "rope_theta": self.rope_theta,
            "rope_scaling": None,
            "hidden_act": "silu",
            "attention_bias": self.attention_bias,
            "tie_word_embeddings": self.tie_word_embeddings,
            "use_sliding_window": self.use_sliding_window,
            "sliding_window": self.sliding_window,
            "max_window_layers": self.max_window_layers,
            "torch_dtype": self.dtype,
            "eos_token_id": eos,
            "bos_token_id": self.bos_token_id,
        }


def read_config_json(model_dir: str) -> Dict[str, Any]:
    path = os.path.join(model_dir, "config.json")
    if not os.path.isdir(model_dir):
        raise ConfigError(f"model path {model_dir!r} is not a directory")
    if not os.path.isfile(path):
        raise ConfigError(f"{model_dir!r} holds no config.json")
    with open(path, "r", encoding="utf-8") as f:
        d = json.load(f)
    if not isinstance(d, dict):
        raise ConfigError(f"{path}: top level is not an object")
    return d


def architecture_name(d: Dict[str, Any], where: str = "config.json") -> str:
    """``architectures[0]``, the key the reference selects the model class by
    (minivllm/models/loader.py:10)."""
    archs = d.get("architectures")
    if archs is None and isinstance(d.get("architecture"), str):
        return d["architecture"]             # configurations that name their one architecture directly
    if not isinstance(archs, (list, tuple)) or not archs or not isinstance(archs[0], str):
        raise ConfigError(f"{where}: 'architectures' must be a non-empty list of names")
    return archs[0]


# ---------------------------------------------------------------------------------------
# Bolapel
# ---------------------------------------------------------------------------------------
def _section(d: Dict[str, Any], key: str, where: str, optional: bool = False) -> Optional[Dict[str, Any]]:
    v = d.get(key)
    if v is None:
        if optional:
            return None
        raise ConfigError(f"{where}: required section '{key}' is missing")
    if not isinstance(v, dict):
        raise ConfigError(f"{where}: '{key}' must be an object, got {v!r}")
    return v


@dataclass(frozen=True)
class BolapelLayer:
    """One entry of Bolapel's ``layers``. ``type`` is "general_delta" (heads, dim) or "attention"
    (heads, kv_heads, dim, vdim, scale, the chunk of its mask, the rotation's dims and base, and
    ``kv_from``: the layer whose keys and values it reads instead of making its own). ``ff`` is the
    width of the layer's dense feed-forward, None for a layer without one."""
    type: str
    heads: int
    dim: int
    kv_heads: int = 0
    vdim: int = 0
    scale: float = 1.0
    chunk: Optional[int] = None
    rot_dims: int = 0
    rot_base: float = 10000.0
    kv_from: Optional[int] = None
    ff: Optional[int] = None
    # general_delta: rows of the first of the two small matrices behind the decay. config.json need not
    # state it (key "rank"); the stored tensor's shape does, and the loader fills it in from there
    decay_rank: Optional[int] = None

    def mixer_dict(self) -> Dict[str, Any]:
        if self.type == "general_delta":
            m = {"heads": self.heads, "dim": self.dim}
            if self.decay_rank is not None:
                m["rank"] = self.decay_rank
            return m
        m: Dict[str, Any] = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim,
                             "scale": self.scale}
        if self.chunk is not None:
            m["mask"] = {"size": self.chunk}
        if self.rot_dims:
            m["rot"] = {"dims": self.rot_dims, "base": self.rot_base}
        if self.kv_from is not None:
            m["kv_from"] = self.kv_from
        return m


@dataclass(frozen=True)
class BolapelConfig(ModelConfig):
    """Bolapel: a decoder whose layers are listed one by one in ``layers``; each has a mixer (a
    generalised delta rule with a matrix state per head, or sigmoid-weighted attention inside chunks
    of the sequence, possibly on another layer's keys and values) and optionally a dense gated
    feed-forward, every sublayer with a norm in front and behind and a token shift in front of the
    mixer. Keys: ``vocab``, ``width``, ``layers``, ``norm.eps``, ``logit_softcap``; the architecture
    is named by ``architecture``. The model states no longest sequence; ``max_position_embeddings``
    here only bounds what an engine may be asked to serve."""

    architecture: ClassVar[str] = "Bolapel"

    vocab_size: int = 0
    hidden_size: int = 0
    layers: Tuple[BolapelLayer, ...] = ()
    norm_eps: float = 1e-5
    logit_softcap: Optional[float] = None
    max_position_embeddings: int = 1 << 24
    dtype: str = "bfloat16"
    eos_token_ids: Tuple[int, ...] = ()

    @classmethod
    def from_dict(cls, d: Dict[str, Any], where: str = "config.json") -> "BolapelConfig":
        raw_layers = d.get("layers")
        if not isinstance(raw_layers, (list, tuple)) or not raw_layers:
            raise ConfigError(f"{where}: 'layers' must be a non-empty list")
        layers = []
        for i, entry in enumerate(raw_layers):
            lw = f"{where}: layers[{i}]"
            if not isinstance(entry, dict):
                raise ConfigError(f"{lw} must be an object")
            kind = entry.get("type")
            m = _section(entry, "mixer", lw)
            mw = lw + ".mixer"
            mlp = _section(entry, "mlp", lw, optional=True)
            ff = None
            if mlp is not None:
                if mlp.get("kind", "dense") != "dense":
                    raise ConfigError(f"{lw}.mlp: kind {mlp.get('kind')!r} is not supported (dense only)")
                ff = _require(mlp, "ff", int, lw + ".mlp")
            if kind == "general_delta":
                rank = m.get("rank")
                layers.append(BolapelLayer(type=kind, heads=_require(m, "heads", int, mw),
                                           dim=_require(m, "dim", int, mw), ff=ff,
                                           decay_rank=None if rank is None else _typed(rank, "rank", int, mw)))
            elif kind == "attention":
                mask = _section(m, "mask", mw, optional=True)
                rot = _section(m, "rot", mw, optional=True)
                heads = _require(m, "heads", int, mw)
                dim = _require(m, "dim", int, mw)
                kv_heads = m.get("kv_heads")
                vdim = m.get("vdim")
                kv_from = m.get("kv_from")
                layers.append(BolapelLayer(
                    type=kind, heads=heads, dim=dim,
                    kv_heads=heads if kv_heads is None else _typed(kv_heads, "kv_heads", int, mw),
                    vdim=dim if vdim is None else _typed(vdim, "vdim", int, mw),
                    scale=_require(m, "scale", float, mw),
                    chunk=None if mask is None else _require(mask, "size", int, mw + ".mask"),
                    rot_dims=0 if rot is None else _require(rot, "dims", int, mw + ".rot"),
                    rot_base=10000.0 if rot is None else _require(rot, "base", float, mw + ".rot"),
                    kv_from=None if kv_from is None else _typed(kv_from, "kv_from", int, mw), ff=ff))
            else:
                raise ConfigError(f"{lw}: layer type {kind!r} is not supported (general_delta, attention)")
        norm = _section(d, "norm", where)
        cap = d.get("logit_softcap")
        dtype = d.get("dtype", d.get("torch_dtype", "bfloat16")) or "bfloat16"
        if str(dtype) not in _DTYPE_NAMES:
            raise ConfigError(f"{where}: unknown dtype {dtype!r}")
        eos = d.get("eos_token_id")
        eos_ids: Tuple[int, ...] = ()
        if isinstance(eos, int) and not isinstance(eos, bool):
            eos_ids = (eos,)
        elif isinstance(eos, (list, tuple)) and all(isinstance(e, int) for e in eos):
            eos_ids = tuple(eos)
        elif eos is not None:
            raise ConfigError(f"{where}: eos_token_id must be an integer or a list of integers, got {eos!r}")
        max_pos = d.get("max_position_embeddings")
        cfg = cls(
            vocab_size=_require(d, "vocab", int, where),
            hidden_size=_require(d, "width", int, where),
            layers=tuple(layers),
            norm_eps=_require(norm, "eps", float, where + ".norm"),
            logit_softcap=None if cap is None else _typed(cap, "logit_softcap", float, where),
            max_position_embeddings=(1 << 24) if max_pos is None else _typed(max_pos, "max_position_embeddings", int, where),
            dtype=_DTYPE_NAMES[str(dtype)],
            eos_token_ids=eos_ids,
        )
        cfg.validate(where)
        return cfg

    def validate(self, where: str = "config") -> None:
        if self.vocab_size <= 0 or self.hidden_size <= 0:
            raise ConfigError(f"{where}: vocab and width must be positive")
        if self.norm_eps <= 0:
            raise ConfigError(f"{where}: norm.eps must be positive, got {self.norm_eps}")
        if self.logit_softcap is not None and self.logit_softcap <= 0:
            raise ConfigError(f"{where}: logit_softcap must be positive, got {self.logit_softcap}")
        for i, l in enumerate(self.layers):
            lw = f"{where}: layers[{i}]"
            if l.heads <= 0 or l.dim <= 0:
                raise ConfigError(f"{lw}: heads and dim must be positive")
            if l.ff is not None and l.ff <= 0:
                raise ConfigError(f"{lw}: mlp.ff must be positive")
            if l.type != "attention":
                continue
            if l.kv_heads <= 0 or l.vdim <= 0 or l.heads % l.kv_heads:
                raise ConfigError(f"{lw}: {l.heads} heads are not a multiple of {l.kv_heads} kv_heads (or vdim <= 0)")
            if l.chunk is not None and l.chunk < 1:
                raise ConfigError(f"{lw}: mask.size must be >= 1, got {l.chunk}")
            if l.rot_dims < 0 or l.rot_dims % 2 or l.rot_dims > l.dim:
                raise ConfigError(f"{lw}: rot.dims {l.rot_dims} must be even and at most dim {l.dim}")
            if l.rot_dims and l.rot_base <= 0:
                raise ConfigError(f"{lw}: rot.base must be positive")
            if l.kv_from is not None:
                j = l.kv_from
                if not (0 <= j < i) or self.layers[j].type != "attention" or self.layers[j].kv_from is not None:
                    raise ConfigError(f"{lw}: kv_from {j} must name an earlier attention layer with keys of its own")
                o = self.layers[j]
                if (o.kv_heads, o.dim, o.vdim, o.rot_dims, o.rot_base) != (l.kv_heads, l.dim, l.vdim, l.rot_dims, l.rot_base):
                    raise ConfigError(f"{lw}: kv_from {j} has other key/value heads, sizes or rotation than this layer")

    def to_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {
            "architecture": self.architecture,
            "layers": [{"type": l.type, "mixer": l.mixer_dict(),
                        "mlp": None if l.ff is None else {"kind": "dense", "ff": l.ff}} for l in self.layers],
            "norm": {"eps": self.norm_eps},
            "vocab": self.vocab_size,
            "width": self.hidden_size,
            "torch_dtype": self.dtype,
        }
        if self.logit_softcap is not None:
            d["logit_softcap"] = self.logit_softcap
        if self.eos_token_ids:
            d["eos_token_id"] = list(self.eos_token_ids) if len(self.eos_token_ids) > 1 else self.eos_token_ids[0]
        if self.max_position_embeddings != (1 << 24):
            d["max_position_embeddings"] = self.max_position_embeddings
        return d


# ---------------------------------------------------------------------------------------
# Dutilix
# ---------------------------------------------------------------------------------------
@dataclass(frozen=True)
class DutilixMixer:
    """The mixer of one Dutilix layer. ``type`` selects which fields count:

    delta             heads, kv_heads (query/key groups), dim (query/key size), vdim, conv (taps)
    mlstm             heads, dim, vdim, gate_cap
    latent_attention  heads, dim (unrotated query/key size), rot_dim, vdim, q_rank, kv_rank, scale, rot_base
    """
    type: str
    heads: int
    dim: int
    vdim: int
    kv_heads: int = 0
    conv: int = 1
    gate_cap: float = 0.0
    rot_dim: int = 0
    rot_base: float = 10000.0
    q_rank: int = 0
    kv_rank: int = 0
    scale: float = 1.0

    def to_dict(self) -> Dict[str, Any]:
        if self.type == "delta":
            return {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim, "conv": self.conv}
        if self.type == "mlstm":
            return {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "gate_cap": self.gate_cap}
        return {"heads": self.heads, "dim": self.dim, "rot_dim": self.rot_dim, "vdim": self.vdim, "q_rank": self.q_rank,
                "kv_rank": self.kv_rank, "scale": self.scale, "rot": {"dims": self.rot_dim, "base": self.rot_base}}


@dataclass(frozen=True)
class DutilixFeedForward:
    """``kind`` "dense": a gated pair of width ``ff``. "moe": ``experts`` gated pairs of width ``ff`` and ``identity``
    identity experts behind them, ``top`` used per token, chosen within ``groups_keep`` of ``groups`` groups."""
    kind: str
    ff: int
    experts: int = 0
    identity: int = 0
    top: int = 0
    groups: int = 1
    groups_keep: int = 1

    def to_dict(self) -> Dict[str, Any]:
        if self.kind == "dense":
            return {"kind": "dense", "ff": self.ff}
        return {"kind": "moe", "expert": {"ff": self.ff},
                "router": {"experts": self.experts, "identity": self.identity, "top": self.top,
                           "groups": {"count": self.groups, "keep": self.groups_keep}}}


@dataclass(frozen=True)
class DutilixLayer:
    mixer: DutilixMixer
    mlp: Optional[DutilixFeedForward] = None


@dataclass(frozen=True)
class DutilixConfig(ModelConfig):
    """Dutilix: a pre-norm decoder whose ``layers`` are listed one by one; each has a mixer (``type``:
    a gated delta rule, an mLSTM matrix memory, or softmax attention over a cached latent) and a
    feed-forward (dense, a mixture of experts, or none). Keys: ``vocab``, ``width``, ``layers``,
    ``norm.eps``, ``logit_scale``; the architecture is named by ``architecture``."""

    architecture: ClassVar[str] = "Dutilix"

    vocab_size: int = 0
    hidden_size: int = 0
    layers: Tuple[DutilixLayer, ...] = ()
    norm_eps: float = 1e-6
    logit_scale: float = 1.0
    max_position_embeddings: int = 1 << 24
    dtype: str = "bfloat16"
    eos_token_ids: Tuple[int, ...] = ()

    @classmethod
    def from_dict(cls, d: Dict[str, Any], where: str = "config.json") -> "DutilixConfig":
        raw_layers = d.get("layers")
        if not isinstance(raw_layers, (list, tuple)) or not raw_layers:
            raise ConfigError(f"{where}: 'layers' must be a non-empty list")
        layers = []
        for i, entry in enumerate(raw_layers):
            lw = f"{where}: layers[{i}]"
            if not isinstance(entry, dict):
                raise ConfigError(f"{lw} must be an object")
            kind = entry.get("type")
            m = _section(entry, "mixer", lw)
            mw = lw + ".mixer"
            heads = _require(m, "heads", int, mw)
            dim = _require(m, "dim", int, mw)
            vdim = _require(m, "vdim", int, mw)
            if kind == "delta":
                kv_heads = m.get("kv_heads")
                conv = m.get("conv")
                # (taps not stated: the stored taps' shape states them, the loader fills them in; 0 stands for "not yet known")
                mixer = DutilixMixer(type=kind, heads=heads, dim=dim, vdim=vdim,
                                     kv_heads=heads if kv_heads is None else _typed(kv_heads, "kv_heads", int, mw),
                                     conv=0 if conv is None else _typed(conv, "conv", int, mw))
            elif kind == "mlstm":
                mixer = DutilixMixer(type=kind, heads=heads, dim=dim, vdim=vdim,
                                     gate_cap=_require(m, "gate_cap", float, mw))
            elif kind == "latent_attention":
                rot = _section(m, "rot", mw, optional=True)
                rot_dim = _typed(m.get("rot_dim", 0) or 0, "rot_dim", int, mw)
                if rot is not None and _require(rot, "dims", int, mw + ".rot") != rot_dim:
                    raise ConfigError(f"{mw}: rot.dims {rot.get('dims')} differs from rot_dim {rot_dim}; the rotated part "
                                      f"is rotated as a whole")
                if rot is None and rot_dim:
                    raise ConfigError(f"{mw}: rot_dim {rot_dim} without a 'rot' section")
                q_rank, kv_rank, scale = m.get("q_rank"), m.get("kv_rank"), m.get("scale")
                # (ranks not stated: the stored norm weights' shapes state them, the loader fills them in)
                mixer = DutilixMixer(type=kind, heads=heads, dim=dim, vdim=vdim, rot_dim=rot_dim,
                                     rot_base=10000.0 if rot is None else _require(rot, "base", float, mw + ".rot"),
                                     q_rank=0 if q_rank is None else _typed(q_rank, "q_rank", int, mw),
                                     kv_rank=0 if kv_rank is None else _typed(kv_rank, "kv_rank", int, mw),
                                     scale=(dim + rot_dim) ** -0.5 if scale is None else _typed(scale, "scale", float, mw))
            else:
                raise ConfigError(f"{lw}: layer type {kind!r} is not supported (delta, mlstm, latent_attention)")
            mlp = _section(entry, "mlp", lw, optional=True)
            ff = None
            if mlp is not None:
                pw = lw + ".mlp"
                mk = mlp.get("kind", "dense")
                if mk == "dense":
                    ff = DutilixFeedForward(kind="dense", ff=_require(mlp, "ff", int, pw))
                elif mk == "moe":
                    expert = _section(mlp, "expert", pw)
                    router = _section(mlp, "router", pw)
                    groups = _section(router, "groups", pw + ".router", optional=True)
                    identity = router.get("identity")
                    ff = DutilixFeedForward(
                        kind="moe", ff=_require(expert, "ff", int, pw + ".expert"),
                        experts=_require(router, "experts", int, pw + ".router"),
                        identity=0 if identity is None else _typed(identity, "identity", int, pw + ".router"),
                        top=_require(router, "top", int, pw + ".router"),
                        groups=1 if groups is None else _require(groups, "count", int, pw + ".router.groups"),
                        groups_keep=1 if groups is None else _require(groups, "keep", int, pw + ".router.groups"))
                else:
                    raise ConfigError(f"{pw}: kind {mk!r} is not supported (dense, moe)")
            layers.append(DutilixLayer(mixer=mixer, mlp=ff))
        norm = _section(d, "norm", where)
        scale = d.get("logit_scale")
        dtype = d.get("dtype", d.get("torch_dtype", "bfloat16")) or "bfloat16"
        if str(dtype) not in _DTYPE_NAMES:
            raise ConfigError(f"{where}: unknown dtype {dtype!r}")
        eos = d.get("eos_token_id")
        eos_ids: Tuple[int, ...] = ()
        if isinstance(eos, int) and not isinstance(eos, bool):
            eos_ids = (eos,)
        elif isinstance(eos, (list, tuple)) and all(isinstance(e, int) for e in eos):
            eos_ids = tuple(eos)
        elif eos is not None:
            raise ConfigError(f"{where}: eos_token_id must be an integer or a list of integers, got {eos!r}")
        max_pos = d.get("max_position_embeddings")
        cfg = cls(
            vocab_size=_require(d, "vocab", int, where),
            hidden_size=_require(d, "width", int, where),
            layers=tuple(layers),
            norm_eps=_require(norm, "eps", float, where + ".norm"),
            logit_scale=1.0 if scale is None else _typed(scale, "logit_scale", float, where),
            max_position_embeddings=(1 << 24) if max_pos is None else _typed(max_pos, "max_position_embeddings", int, where),
            dtype=_DTYPE_NAMES[str(dtype)],
            eos_token_ids=eos_ids,
        )
        cfg.validate(where)
        return cfg

    def validate(self, where: str = "config") -> None:
        if self.vocab_size <= 0 or self.hidden_size <= 0:
            raise ConfigError(f"{where}: vocab and width must be positive")
        if self.norm_eps <= 0:
            raise ConfigError(f"{where}: norm.eps must be positive, got {self.norm_eps}")
        for i, l in enumerate(self.layers):
            lw = f"{where}: layers[{i}]"
            m = l.mixer
            if m.heads <= 0 or m.dim <= 0 or m.vdim <= 0:
                raise ConfigError(f"{lw}: heads, dim and vdim must be positive")
            if m.type == "delta":
                if m.kv_heads <= 0 or m.heads % m.kv_heads:
                    raise ConfigError(f"{lw}: {m.heads} heads are not a multiple of {m.kv_heads} kv_heads")
                if m.conv < 0:
                    raise ConfigError(f"{lw}: conv must be >= 1, got {m.conv}")
            elif m.type == "mlstm":
                if not m.gate_cap > 0:
                    raise ConfigError(f"{lw}: gate_cap must be positive, got {m.gate_cap}")
            else:
                if m.q_rank < 0 or m.kv_rank < 0:
                    raise ConfigError(f"{lw}: q_rank and kv_rank must be positive")
                if m.rot_dim < 0 or m.rot_dim % 2:
                    raise ConfigError(f"{lw}: rot_dim {m.rot_dim} must be even and >= 0")
                if m.rot_dim and m.rot_base <= 0:
                    raise ConfigError(f"{lw}: rot.base must be positive")
            f = l.mlp
            if f is None:
                continue
            if f.ff <= 0:
                raise ConfigError(f"{lw}: the feed-forward width must be positive")
            if f.kind == "moe":
                total = f.experts + f.identity
                if f.experts < 0 or f.identity < 0 or total < 1:
                    raise ConfigError(f"{lw}: a router needs at least one expert")
                if f.groups < 1 or total % f.groups or not (1 <= f.groups_keep <= f.groups):
                    raise ConfigError(f"{lw}: {total} router outputs do not form {f.groups} equal groups of which "
                                      f"{f.groups_keep} are kept")
                if not (1 <= f.top <= total // f.groups * f.groups_keep):
                    raise ConfigError(f"{lw}: top {f.top} exceeds the experts that can be chosen")

    def to_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {
            "architecture": self.architecture,
            "layers": [{"type": l.mixer.type, "mixer": l.mixer.to_dict(), "mlp": None if l.mlp is None else l.mlp.to_dict()}
                       for l in self.layers],
            "norm": {"eps": self.norm_eps},
            "logit_scale": self.logit_scale,
            "vocab": self.vocab_size,
            "width": self.hidden_size,
            "torch_dtype": self.dtype,
        }
        if self.eos_token_ids:
            d["eos_token_id"] = list(self.eos_token_ids) if len(self.eos_token_ids) > 1 else self.eos_token_ids[0]
        if self.max_position_embeddings != (1 << 24):
            d["max_position_embeddings"] = self.max_position_embeddings
        return d


# ---------------------------------------------------------------------------------------
# Zedudra
# ---------------------------------------------------------------------------------------
@dataclass(frozen=True)
class ZedudraMixer:
    """The attention of one Zedudra layer: ``heads`` query heads on ``kv_heads`` key/value heads of size ``dim``
    (the values are the keys, so ``vdim`` equals ``dim``), a window of ``window`` positions (the query's own among
    them) beside the sequence's first ``keep_first``, rotation of the first ``rot_dims`` channels of a head."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: int
    keep_first: int = 0
    rot_dims: int = 0
    rot_base: float = 10000.0

    def to_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {"heads": self.heads, "kv_heads": self.kv_heads, "dim": self.dim, "vdim": self.vdim,
                             "scale": self.scale, "mask": {"size": self.window, "keep_first": self.keep_first}}
        if self.rot_dims:
            d["rot"] = {"dims": self.rot_dims, "base": self.rot_base}
        return d


@dataclass(frozen=True)
class ZedudraFeedForward:
    """``kind`` "dense": two projections of width ``ff`` around the xIELU activation. "moe": ``experts`` clamped gated
    pairs of width ``ff`` (clamp at ``limit``), ``top`` used per token, chosen within ``groups_keep`` of ``groups`` groups."""
    kind: str
    ff: int
    limit: float = 0.0
    experts: int = 0
    top: int = 0
    groups: int = 1
    groups_keep: int = 1

    def to_dict(self) -> Dict[str, Any]:
        if self.kind == "dense":
            return {"kind": "dense", "ff": self.ff}
        return {"kind": "moe", "expert": {"ff": self.ff, "limit": self.limit},
                "router": {"experts": self.experts, "top": self.top, "groups": {"count": self.groups, "keep": self.groups_keep}}}


@dataclass(frozen=True)
class ZedudraLayer:
    mixer: ZedudraMixer
    mlp: Optional[ZedudraFeedForward] = None
    weights_of: Optional[int] = None       # the layer whose tensors this one uses (it keeps a cache and state of its own)


@dataclass(frozen=True)
class ZedudraConfig(ModelConfig):
    """Zedudra: a decoder whose ``layers`` are listed one by one. Each has a norm in groups in front of and behind
    its attention and its feed-forward, a short causal convolution added to the attention's input (``canon.taps``),
    softmax attention over a window and the sequence's first positions with the keys as values and a gate per head,
    and a dense (xIELU) or routed feed-forward, or none. A layer may use another layer's tensors (``weights_of``).
    Keys: ``vocab``, ``width``, ``layers``, ``norm.eps``, ``norm.groups``, ``canon.taps``, ``embedding.scale``."""

    architecture: ClassVar[str] = "Zedudra"

    vocab_size: int = 0
    hidden_size: int = 0
    layers: Tuple[ZedudraLayer, ...] = ()
    norm_eps: float = 1e-6
    norm_groups: int = 1
    conv_taps: int = 0                     # 0: no convolution in front of the mixers
    embedding_scale: float = 1.0
    max_position_embeddings: int = 1 << 24
    dtype: str = "bfloat16"
    eos_token_ids: Tuple[int, ...] = ()

    @classmethod
    def from_dict(cls, d: Dict[str, Any], where: str = "config.json") -> "ZedudraConfig":
        raw_layers = d.get("layers")
        if not isinstance(raw_layers, (list, tuple)) or not raw_layers:
            raise ConfigError(f"{where}: 'layers' must be a non-empty list")
        layers = []
        for i, entry in enumerate(raw_layers):
            lw = f"{where}: layers[{i}]"
            if not isinstance(entry, dict):
                raise ConfigError(f"{lw} must be an object")
            if entry.get("type") != "attention":
                raise ConfigError(f"{lw}: layer type {entry.get('type')!r} is not supported (attention)")
            m = _section(entry, "mixer", lw)
            mw = lw + ".mixer"
            heads = _require(m, "heads", int, mw)
            dim = _require(m, "dim", int, mw)
            kv_heads, vdim, scale = m.get("kv_heads"), m.get("vdim"), m.get("scale")
            mask = _section(m, "mask", mw)
            rot = _section(m, "rot", mw, optional=True)
            keep = mask.get("keep_first")
            mixer = ZedudraMixer(
                heads=heads, dim=dim,
                kv_heads=heads if kv_heads is None else _typed(kv_heads, "kv_heads", int, mw),
                vdim=dim if vdim is None else _typed(vdim, "vdim", int, mw),
                scale=dim ** -0.5 if scale is None else _typed(scale, "scale", float, mw),
                window=_require(mask, "size", int, mw + ".mask"),
                keep_first=0 if keep is None else _typed(keep, "keep_first", int, mw + ".mask"),
                rot_dims=0 if rot is None else _require(rot, "dims", int, mw + ".rot"),
                rot_base=10000.0 if rot is None else _require(rot, "base", float, mw + ".rot"))
            mlp = _section(entry, "mlp", lw, optional=True)
            ff = None
            if mlp is not None:
                pw = lw + ".mlp"
                mk = mlp.get("kind", "dense")
                if mk == "dense":
                    ff = ZedudraFeedForward(kind="dense", ff=_require(mlp, "ff", int, pw))
                elif mk == "moe":
                    expert = _section(mlp, "expert", pw)
                    router = _section(mlp, "router", pw)
                    groups = _section(router, "groups", pw + ".router", optional=True)
                    ff = ZedudraFeedForward(
                        kind="moe", ff=_require(expert, "ff", int, pw + ".expert"),
                        limit=_require(expert, "limit", float, pw + ".expert"),
                        experts=_require(router, "experts", int, pw + ".router"),
                        top=_require(router, "top", int, pw + ".router"),
                        groups=1 if groups is None else _require(groups, "count", int, pw + ".router.groups"),
                        groups_keep=1 if groups is None else _require(groups, "keep", int, pw + ".router.groups"))
                else:
                    raise ConfigError(f"{pw}: kind {mk!r} is not supported (dense, moe)")
            shared = entry.get("weights_of")
            layers.append(ZedudraLayer(mixer=mixer, mlp=ff,
                                       weights_of=None if shared is None else _typed(shared, "weights_of", int, lw)))
        norm = _section(d, "norm", where)
        groups = norm.get("groups")
        canon = _section(d, "canon", where, optional=True)
        emb = _section(d, "embedding", where, optional=True)
        emb_scale = None if emb is None else emb.get("scale")
        dtype = d.get("dtype", d.get("torch_dtype", "bfloat16")) or "bfloat16"
        if str(dtype) not in _DTYPE_NAMES:
            raise ConfigError(f"{where}: unknown dtype {dtype!r}")
        eos = d.get("eos_token_id")
        eos_ids: Tuple[int, ...] = ()
        if isinstance(eos, int) and not isinstance(eos, bool):
            eos_ids = (eos,)
        elif isinstance(eos, (list, tuple)) and all(isinstance(e, int) for e in eos):
            eos_ids = tuple(eos)
        elif eos is not None:
            raise ConfigError(f"{where}: eos_token_id must be an integer or a list of integers, got {eos!r}")
        max_pos = d.get("max_position_embeddings")
        cfg = cls(
            vocab_size=_require(d, "vocab", int, where),
            hidden_size=_require(d, "width", int, where),
            layers=tuple(layers),
            norm_eps=_require(norm, "eps", float, where + ".norm"),
            norm_groups=1 if groups is None else _typed(groups, "groups", int, where + ".norm"),
            conv_taps=0 if canon is None else _require(canon, "taps", int, where + ".canon"),
            embedding_scale=1.0 if emb_scale is None else _typed(emb_scale, "scale", float, where + ".embedding"),
            max_position_embeddings=(1 << 24) if max_pos is None else _typed(max_pos, "max_position_embeddings", int, where),
            dtype=_DTYPE_NAMES[str(dtype)],
            eos_token_ids=eos_ids,
        )
        cfg.validate(where)
        return cfg

    def validate(self, where: str = "config") -> None:
        if self.vocab_size <= 0 or self.hidden_size <= 0:
            raise ConfigError(f"{where}: vocab and width must be positive")
        if self.norm_eps <= 0:
            raise ConfigError(f"{where}: norm.eps must be positive, got {self.norm_eps}")
        if self.norm_groups < 1 or self.hidden_size % self.norm_groups:
            raise ConfigError(f"{where}: a width of {self.hidden_size} does not form {self.norm_groups} equal norm groups")
        if self.conv_taps < 0 or self.conv_taps > 16:
            raise ConfigError(f"{where}: canon.taps must lie in 1..16, got {self.conv_taps}")
        for i, l in enumerate(self.layers):
            lw = f"{where}: layers[{i}]"
            m = l.mixer
            if m.heads <= 0 or m.dim <= 0 or m.kv_heads <= 0 or m.heads % m.kv_heads:
                raise ConfigError(f"{lw}: {m.heads} heads of {m.dim} are not a multiple of {m.kv_heads} kv_heads")
            if m.vdim != m.dim:
                raise ConfigError(f"{lw}: the values are the keys, so vdim {m.vdim} must equal dim {m.dim}")
            if m.window < 1 or m.keep_first < 0:
                raise ConfigError(f"{lw}: mask.size must be >= 1 and mask.keep_first >= 0")
            if m.rot_dims < 0 or m.rot_dims % 2 or m.rot_dims > m.dim:
                raise ConfigError(f"{lw}: rot.dims {m.rot_dims} must be even and at most dim {m.dim}")
            if m.rot_dims and m.rot_base <= 0:
                raise ConfigError(f"{lw}: rot.base must be positive")
            f = l.mlp
            if f is not None:
                if f.ff <= 0:
                    raise ConfigError(f"{lw}: the feed-forward width must be positive")
                if f.kind == "moe":
                    if f.experts < 1 or not f.limit > 0:
                        raise ConfigError(f"{lw}: a router needs at least one expert and a positive expert.limit")
                    if f.groups < 1 or f.experts % f.groups or not (1 <= f.groups_keep <= f.groups):
                        raise ConfigError(f"{lw}: {f.experts} experts do not form {f.groups} equal groups of which "
                                          f"{f.groups_keep} are kept")
                    if not (1 <= f.top <= f.experts // f.groups * f.groups_keep):
                        raise ConfigError(f"{lw}: top {f.top} exceeds the experts that can be chosen")
            if l.weights_of is not None:
                j = self.owner_of(i, lw)
                if (self.layers[j].mixer, self.layers[j].mlp) != (l.mixer, l.mlp):
                    raise ConfigError(f"{lw}: weights_of {j} names a layer with other sizes or constants than this one")

    def owner_of(self, i: int, where: str = "layers") -> int:
        """The layer whose tensors layer ``i`` uses: itself, or the end of its chain of ``weights_of`` (a layer may
        name one that itself uses another's; the chain may point backwards or forwards but must end)."""
        seen = {i}
        while self.layers[i].weights_of is not None:
            j = self.layers[i].weights_of
            if not (0 <= j < len(self.layers)) or j in seen:
                raise ConfigError(f"{where}: weights_of {j} must name another layer of the model, and the chain must end "
                                  f"at a layer with tensors of its own")
            seen.add(j)
            i = j
        return i

    def to_dict(self) -> Dict[str, Any]:
        layers = []
        for l in self.layers:
            e: Dict[str, Any] = {"type": "attention", "mixer": l.mixer.to_dict(), "mlp": None if l.mlp is None else l.mlp.to_dict()}
            if l.weights_of is not None:
                e["weights_of"] = l.weights_of
            layers.append(e)
        d: Dict[str, Any] = {
            "architecture": self.architecture,
            "layers": layers,
            "norm": {"eps": self.norm_eps, "groups": self.norm_groups},
            "embedding": {"scale": self.embedding_scale},
            "vocab": self.vocab_size,
            "width": self.hidden_size,
            "torch_dtype": self.dtype,
        }
        if self.conv_taps:
            d["canon"] = {"taps": self.conv_taps}
        if self.eos_token_ids:
            d["eos_token_id"] = list(self.eos_token_ids) if len(self.eos_token_ids) > 1 else self.eos_token_ids[0]
        if self.max_position_embeddings != (1 << 24):
            d["max_position_embeddings"] = self.max_position_embeddings
        return d


# ---------------------------------------------------------------------------------------
# Furanex
# ---------------------------------------------------------------------------------------
UNSTATED = -1          # a size that config.json leaves to the shapes of the stored tensors (``furanex_complete`` fills it in)


def _size(d: Dict[str, Any], key: str, where: str) -> int:
    """An integer size of config.json, or UNSTATED when the key is absent."""
    v = d.get(key)
    return UNSTATED if v is None else _typed(v, key, int, where)


@dataclass(frozen=True)
class FuranexRotation:
    """Rotation by position over the first ``dims`` channels; ``stretch`` = (factor, original, fast, slow) slows the
    low frequencies down for contexts longer than ``original`` (None: plain frequencies)."""
    dims: int
    base: float
    stretch: Optional[Tuple[float, float, float, float]] = None

    def to_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {"dims": self.dims, "base": self.base}
        if self.stretch is not None:
            d["scaling"] = dict(zip(("factor", "original", "fast", "slow"), self.stretch))
        return d


@dataclass(frozen=True)
class FuranexMixer:
    """``kind`` "attention": ``heads`` query heads on ``kv_heads`` key/value heads, keys of ``dim`` and values of ``vdim``
    channels, ``v_mix``: the values are shared along the layers. ``kind`` "latent_attention": ``heads`` heads with ``dim``
    unrotated and ``rot_dim`` rotated query/key channels, values of ``vdim``, latents of ``q_rank`` and ``kv_rank``.
    A size may be UNSTATED, and ``scale`` None, until the configuration has been completed."""
    kind: str
    heads: int
    dim: int
    vdim: int
    scale: Optional[float]
    rot: Optional[FuranexRotation] = None
    kv_heads: int = UNSTATED
    v_mix: bool = False
    rot_dim: int = UNSTATED
    q_rank: int = UNSTATED
    kv_rank: int = UNSTATED

    def to_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {"heads": self.heads, "dim": self.dim, "vdim": self.vdim, "scale": self.scale}
        if self.rot is not None:
            d["rot"] = self.rot.to_dict()
        if self.kind == "attention":
            d.update(kv_heads=self.kv_heads, v_mix=self.v_mix)
        else:
            d.update(rot_dim=self.rot_dim, q_rank=self.q_rank, kv_rank=self.kv_rank)
        return {k: v for k, v in d.items() if v is not None and v != UNSTATED}


@dataclass(frozen=True)
class FuranexFeedForward:
    """A mixture of ``experts`` gated pairs of width ``ff`` of which a token uses ``top``, named by a stored table from
    its token id; ``shared_ff`` > 0: a shared expert of that width beside them."""
    ff: int
    experts: int
    top: int
    shared_ff: int = UNSTATED

    def to_dict(self) -> Dict[str, Any]:
        d: Dict[str, Any] = {"kind": "moe", "expert": {}, "router": {}}
        if self.ff != UNSTATED:
            d["expert"]["ff"] = self.ff
        if self.experts != UNSTATED:
            d["router"]["experts"] = self.experts
        if self.top != UNSTATED:
            d["router"]["top"] = self.top
        if self.shared_ff != UNSTATED:
            d["shared"] = {"ff": self.shared_ff} if self.shared_ff else None
        return d


@dataclass(frozen=True)
class FuranexLayer:
    mixer: FuranexMixer
    mlp: Optional[FuranexFeedForward] = None


@dataclass(frozen=True)
class FuranexConfig(ModelConfig):
    """Furanex: a pre-norm decoder on several residual streams (``streams``) whose ``layers`` are listed one by one: grouped
    softmax attention (rotation first, then a unit norm of q and k; values blended with the first such layer's) or
    attention over a cached latent with a gate per head; feed-forwards whose experts a table names by token id, beside a
    shared expert. The embedding is multiplied by ``embedding.scale``; the output head is the embedding's table.
    Keys: ``vocab``, ``width``, ``streams``, ``layers``, ``norm.eps``, ``embedding.scale``. Sizes that config.json leaves
    out are UNSTATED until ``completed`` has filled them in, from the stored tensors' shapes (``models/furanex.py``) or
    with their defaults (``kv_heads`` = heads, ``vdim`` = dim, ``rot_dim`` = rot.dims, no shared expert, one residual)."""

    architecture: ClassVar[str] = "Furanex"

    vocab_size: int = UNSTATED
    hidden_size: int = UNSTATED
    streams: int = UNSTATED                # 0: one plain residual
    layers: Tuple[FuranexLayer, ...] = ()
    norm_eps: float = 1e-6
    embedding_scale: float = 1.0
    max_position_embeddings: int = 1 << 24
    dtype: str = "bfloat16"
    eos_token_ids: Tuple[int, ...] = ()

    @staticmethod
    def _rotation(m: Dict[str, Any], mw: str) -> Optional[FuranexRotation]:
        rot = _section(m, "rot", mw, optional=True)
        if rot is None:
            return None
        rw = mw + ".rot"
        sc = _section(rot, "scaling", rw, optional=True)
        stretch = None
        if sc is not None:
            stretch = tuple(_require(sc, k, float, rw + ".scaling") for k in ("factor", "original", "fast", "slow"))
        return FuranexRotation(dims=_require(rot, "dims", int, rw), base=_require(rot, "base", float, rw), stretch=stretch)

    @classmethod
    def from_dict(cls, d: Dict[str, Any], where: str = "config.json") -> "FuranexConfig":
        raw_layers = d.get("layers")
        if not isinstance(raw_layers, (list, tuple)) or not raw_layers:
            raise ConfigError(f"{where}: 'layers' must be a non-empty list")
        layers = []
        for i, entry in enumerate(raw_layers):
            lw = f"{where}: layers[{i}]"
            if not isinstance(entry, dict):
                raise ConfigError(f"{lw} must be an object")
            kind = entry.get("type")
            if kind not in ("attention", "latent_attention"):
                raise ConfigError(f"{lw}: layer type {kind!r} is not supported (attention, latent_attention)")
            m = _section(entry, "mixer", lw)
            mw = lw + ".mixer"
            scale, v_mix = m.get("scale"), m.get("v_mix")
            if kind == "latent_attention" and v_mix:
                raise ConfigError(f"{mw}: a latent layer caches no values that could be shared along the layers")
            mixer = FuranexMixer(kind=kind, heads=_size(m, "heads", mw), dim=_size(m, "dim", mw), vdim=_size(m, "vdim", mw),
                                 scale=None if scale is None else _typed(scale, "scale", float, mw), rot=cls._rotation(m, mw),
                                 kv_heads=_size(m, "kv_heads", mw), v_mix=False if v_mix is None else _typed(v_mix, "v_mix", bool, mw),
                                 rot_dim=_size(m, "rot_dim", mw), q_rank=_size(m, "q_rank", mw), kv_rank=_size(m, "kv_rank", mw))
            mlp = _section(entry, "mlp", lw, optional=True)
            ff = None
            if mlp is not None:
                pw = lw + ".mlp"
                if mlp.get("kind", "moe") != "moe":
                    raise ConfigError(f"{pw}: kind {mlp.get('kind')!r} is not supported (moe)")
                expert = _section(mlp, "expert", pw, optional=True) or {}
                router = _section(mlp, "router", pw, optional=True) or {}
                if "shared" in mlp:          # stated: a section with its width, or null for none
                    shared = _section(mlp, "shared", pw, optional=True)
                    shared_ff = 0 if shared is None else _size(shared, "ff", pw + ".shared")
                else:
                    shared_ff = UNSTATED
                ff = FuranexFeedForward(ff=_size(expert, "ff", pw + ".expert"), experts=_size(router, "experts", pw + ".router"),
                                        top=_size(router, "top", pw + ".router"), shared_ff=shared_ff)
            layers.append(FuranexLayer(mixer=mixer, mlp=ff))
        norm = _section(d, "norm", where)
        emb = _section(d, "embedding", where, optional=True)
        emb_scale = None if emb is None else emb.get("scale")
        dtype = d.get("dtype", d.get("torch_dtype", "bfloat16")) or "bfloat16"
        if str(dtype) not in _DTYPE_NAMES:
            raise ConfigError(f"{where}: unknown dtype {dtype!r}")
        eos = d.get("eos_token_id")
        eos_ids: Tuple[int, ...] = ()
        if isinstance(eos, int) and not isinstance(eos, bool):
            eos_ids = (eos,)
        elif isinstance(eos, (list, tuple)) and all(isinstance(e, int) for e in eos):
            eos_ids = tuple(eos)
        elif eos is not None:
            raise ConfigError(f"{where}: eos_token_id must be an integer or a list of integers, got {eos!r}")
        max_pos = d.get("max_position_embeddings")
        cfg = cls(
            vocab_size=_size(d, "vocab", where), hidden_size=_size(d, "width", where), streams=_size(d, "streams", where),
            layers=tuple(layers),
            norm_eps=_require(norm, "eps", float, where + ".norm"),
            embedding_scale=1.0 if emb_scale is None else _typed(emb_scale, "scale", float, where + ".embedding"),
            max_position_embeddings=(1 << 24) if max_pos is None else _typed(max_pos, "max_position_embeddings", int, where),
            dtype=_DTYPE_NAMES[str(dtype)],
            eos_token_ids=eos_ids,
        )
        cfg.validate(where)
        return cfg

    def first_mixing_layer(self) -> Optional[int]:
        """The first attention layer whose values are shared along the layers: the others blend its values into theirs."""
        for i, l in enumerate(self.layers):
            if l.mixer.kind == "attention" and l.mixer.v_mix:
                return i
        return None

    def completed(self, sizes=None, where: str = "config") -> "FuranexConfig":
        """The configuration with nothing UNSTATED. ``sizes(name) -> shape or None`` looks a stored tensor's shape up;
        a size that neither config.json nor a shape states takes its default, or is an error when it has none."""
        import dataclasses
        sizes = sizes or (lambda name: None)

        def axis(name: str, k: int) -> Optional[int]:
            shape = sizes(name)
            return None if shape is None or len(shape) <= k else int(shape[k])

        def need(value: int, found: Optional[int], what: str, default: Optional[int] = None) -> int:
            if value != UNSTATED:
                return value
            if found is not None:
                return found
            if default is not None:
                return default
            raise ConfigError(f"{where}: {what} is stated neither in config.json nor by a stored tensor's shape")

        def per(total: Optional[int], count: int) -> Optional[int]:
            return None if total is None or count in (UNSTATED, 0) or total % count else total // count

        vocab = need(self.vocab_size, axis("embed", 0), "vocab")
        width = need(self.hidden_size, axis("embed", 1), "width")
        streams = need(self.streams, axis("l0.hc1.in", 0), "streams", 0)
        layers = []
        for i, l in enumerate(self.layers):
            m, p, lw = l.mixer, f"l{i}.mix.", f"layers[{i}].mixer"
            if m.kind == "attention":
                q_rows, k_rows, v_rows = axis(p + "q", 0), axis(p + "k", 0), axis(p + "v", 0)
                heads = need(m.heads, per(q_rows, m.dim), lw + ".heads")
                dim = need(m.dim, per(q_rows, heads), lw + ".dim")
                kv_heads = need(m.kv_heads, per(k_rows, dim), lw + ".kv_heads", heads)
                vdim = need(m.vdim, per(v_rows, kv_heads), lw + ".vdim", dim)
                m = dataclasses.replace(m, heads=heads, dim=dim, kv_heads=kv_heads, vdim=vdim, rot_dim=0, q_rank=0, kv_rank=0,
                                        scale=dim ** -0.5 if m.scale is None else m.scale)
            else:
                heads = need(m.heads, axis(p + "g", 0), lw + ".heads")
                dim = need(m.dim, per(axis(p + "uk", 0), heads), lw + ".dim")
                vdim = need(m.vdim, per(axis(p + "uv", 0), heads), lw + ".vdim", dim)
                q_rank = need(m.q_rank, axis(p + "dq.norm", 0), lw + ".q_rank")
                kv_rank = need(m.kv_rank, axis(p + "dkv.norm", 0), lw + ".kv_rank")
                rows = axis(p + "dkv", 0)
                rot_dim = need(m.rot_dim, None if rows is None else rows - kv_rank, lw + ".rot_dim", m.rot.dims if m.rot is not None else 0)
                m = dataclasses.replace(m, heads=heads, dim=dim, vdim=vdim, q_rank=q_rank, kv_rank=kv_rank, rot_dim=rot_dim, kv_heads=0,
                                        scale=(dim + rot_dim) ** -0.5 if m.scale is None else m.scale)
            f = l.mlp
            if f is not None:
                y, fw = f"l{i}.mlp.", f"layers[{i}].mlp"
                counted = 0
                while sizes(f"{y}e{counted}.gate") is not None:
                    counted += 1
                f = FuranexFeedForward(ff=need(f.ff, axis(y + "e0.gate", 0), fw + ".expert.ff"),
                                       experts=need(f.experts, counted or None, fw + ".router.experts"),
                                       top=need(f.top, axis(y + "table", 1), fw + ".router.top"),
                                       shared_ff=need(f.shared_ff, axis(y + "shared.gate", 0), fw + ".shared.ff", 0))
            layers.append(FuranexLayer(mixer=m, mlp=f))
        done = dataclasses.replace(self, vocab_size=vocab, hidden_size=width, streams=streams, layers=tuple(layers))
        done.validate(where, final=True)
        return done

    def validate(self, where: str = "config", final: bool = False) -> None:
        """Checks what is stated; with ``final`` nothing may be UNSTATED any more."""
        known = lambda *values: all(v != UNSTATED and v is not None for v in values)
        positive = lambda v: v == UNSTATED or v > 0
        if not positive(self.vocab_size) or not positive(self.hidden_size):
            raise ConfigError(f"{where}: vocab and width must be positive")
        if self.norm_eps <= 0:
            raise ConfigError(f"{where}: norm.eps must be positive, got {self.norm_eps}")
        if self.streams != UNSTATED and not (0 <= self.streams <= 8):
            raise ConfigError(f"{where}: streams must lie in 1..8, got {self.streams}")
        first = self.first_mixing_layer()
        for i, l in enumerate(self.layers):
            lw = f"{where}: layers[{i}]"
            m = l.mixer
            if not all(positive(v) for v in (m.heads, m.dim, m.vdim)) or (m.scale is not None and not m.scale > 0):
                raise ConfigError(f"{lw}: heads, dim, vdim and scale must be positive")
            if m.rot is not None:
                r = m.rot
                if r.dims <= 0 or r.dims % 2 or not r.base > 1:
                    raise ConfigError(f"{lw}: rot.dims {r.dims} must be positive and even, rot.base above 1")
                if r.stretch is not None and not all(v > 0 for v in r.stretch):
                    raise ConfigError(f"{lw}: rot.scaling needs positive factor, original, fast and slow")
            if m.kind == "attention":
                if not positive(m.kv_heads) or (known(m.heads, m.kv_heads) and m.heads % m.kv_heads):
                    raise ConfigError(f"{lw}: {m.heads} heads are not a multiple of {m.kv_heads} kv_heads")
                if m.rot is not None and known(m.dim) and m.rot.dims > m.dim:
                    raise ConfigError(f"{lw}: rot.dims {m.rot.dims} exceeds dim {m.dim}")
                f0 = self.layers[first].mixer if first is not None else None
                if m.v_mix and known(m.kv_heads, m.vdim, f0.kv_heads, f0.vdim) and (f0.kv_heads, f0.vdim) != (m.kv_heads, m.vdim):
                    raise ConfigError(f"{lw}: layers that share their values need the kv_heads and vdim of layer {first}")
            else:
                if not positive(m.q_rank) or not positive(m.kv_rank) or (m.rot_dim != UNSTATED and (m.rot_dim < 0 or m.rot_dim % 2)):
                    raise ConfigError(f"{lw}: q_rank and kv_rank must be positive, rot_dim even and >= 0")
                if known(m.rot_dim) and (m.rot.dims if m.rot is not None else 0) != m.rot_dim:
                    raise ConfigError(f"{lw}: the rotated part has rot_dim {m.rot_dim} channels, so rot.dims must equal it")
            f = l.mlp
            if f is not None:
                if not positive(f.ff) or not positive(f.experts) or not positive(f.top) or f.shared_ff < UNSTATED \
                        or (known(f.top, f.experts) and f.top > f.experts):
                    raise ConfigError(f"{lw}: a mixture needs a positive expert width, experts >= 1 and 1 <= top <= experts")
            if final and not (known(m.heads, m.dim, m.vdim, m.scale, m.kv_heads, m.rot_dim, m.q_rank, m.kv_rank)
                              and (f is None or known(f.ff, f.experts, f.top, f.shared_ff))):
                raise ConfigError(f"{lw}: a size is still not stated")
        if final and not known(self.vocab_size, self.hidden_size, self.streams):
            raise ConfigError(f"{where}: vocab, width or streams is still not stated")

    def to_dict(self) -> Dict[str, Any]:
        layers = [{"type": l.mixer.kind, "mixer": l.mixer.to_dict(), "mlp": None if l.mlp is None else l.mlp.to_dict()}
                  for l in self.layers]
        d: Dict[str, Any] = {
            "architecture": self.architecture,
            "layers": layers,
            "norm": {"eps": self.norm_eps},
            "embedding": {"scale": self.embedding_scale},
            "torch_dtype": self.dtype,
        }
        for key, value in (("vocab", self.vocab_size), ("width", self.hidden_size), ("streams", self.streams)):
            if value != UNSTATED and (key != "streams" or value):
                d[key] = value
        if self.eos_token_ids:
            d["eos_token_id"] = list(self.eos_token_ids) if len(self.eos_token_ids) > 1 else self.eos_token_ids[0]
        if self.max_position_embeddings != (1 << 24):
            d["max_position_embeddings"] = self.max_position_embeddings
        return d
