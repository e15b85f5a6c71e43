"""Zedudra as a plan of parts.

Every layer is a sandwich block (a norm in front of and behind each sublayer) whose norms work in
groups of columns (``parts/norm.py: GroupRMSNorm``) and whose mixer input passes a short causal
convolution over time that is added to it (``parts/block.py``, ``input_conv_taps``). The mixer is
softmax attention over a window and the sequence's first positions, with the keys as values, a
rotation in neighbouring pairs over the first channels of each head and a gate per head
(``parts/attention.py``). The feed-forward is two projections around the xIELU activation
(``parts/mlp.py``) or a mixture of clamped gated experts behind a sigmoid router that picks within
the best groups (``parts/moe.py``); a layer may have none. A layer may use the tensors of an earlier
one: it is then a second call of that layer, with a cache and state of its own. The embedding is
multiplied by a constant.

Tensor names on disk: ``embed``, ``head``, ``final.norm``; per layer i ``l<i>.norm1``, ``.norm1b``,
``.norm2``, ``.norm2b``, ``.canon1``, ``l<i>.mix.{q,k,g,o}`` and ``l<i>.mlp.{up,down,act}`` or
``l<i>.mlp.{router,e<j>.gate,e<j>.up,e<j>.down}``.
"""
from __future__ import annotations

from typing import Dict, FrozenSet

from ..config.model_config import ZedudraConfig
from ..parts.attention import AttentionSpec
from ..parts.block import SandwichBlock, SandwichBlockSpec
from ..parts.mlp import XIELUSpec
from ..parts.moe import RoutedExpertsSpec
from ..parts.norm import GroupRMSNormSpec
from ..parts.plan import Call, EmbeddingSpec, HeadSpec, LayerPlan, ModelPlan, TensorLocation
from ..parts.rope import RotarySpec
from .registry import Architecture, register_architecture

GATE_SLOPE = 1.702        # an expert's gate is g * sigmoid(GATE_SLOPE * g)


def zedudra_plan(config: ZedudraConfig) -> ModelPlan:
    hid = config.hidden_size
    norm = GroupRMSNormSpec(size=hid, eps=config.norm_eps, groups=config.norm_groups)
    block = SandwichBlockSpec(hidden_size=hid, input_conv_taps=config.conv_taps)
    layers, calls = [], []
    # config layer with tensors of its own -> layer of the plan
    index_of: Dict[int, int] = {i: k for k, i in enumerate(_owners(config))}
    for i, l in enumerate(config.layers):
        if l.weights_of is not None:
            calls.append(Call(layer=index_of[config.owner_of(i)]))
            continue
        m = l.mixer
        rope = RotarySpec(rotary_dim=m.rot_dims, theta=m.rot_base, interleaved=True) if m.rot_dims else None
        # the configuration counts the query's own position into the window, the part counts the positions left of it
        mixer = AttentionSpec(hidden_size=hid, num_heads=m.heads, num_kv_heads=m.kv_heads, head_dim=m.dim, scale=m.scale,
                              qk_norm=False, bias=False, window=m.window - 1, position=rope, head_gate=True,
                              keep_first=m.keep_first, value_from_key=True)
        f = l.mlp
        if f is None:
            ffn = None
        elif f.kind == "dense":
            ffn = XIELUSpec(hidden_size=hid, intermediate_size=f.ff)
        else:
            ffn = RoutedExpertsSpec(hidden_size=hid, expert_size=f.ff, num_experts=f.experts, top=f.top, groups=f.groups,
                                    keep_groups=f.groups_keep, correction=False, scoring="sigmoid", group_worth="top2",
                                    normalize=False, activation="clamped", limit=f.limit, gate_slope=GATE_SLOPE)
        slots = SandwichBlock.slots_for(ffn is not None)
        assert index_of[i] == len(layers)
        layers.append(LayerPlan(block=block, mixer=mixer, ffn=ffn, norms=tuple((s, norm) for s in slots)))
        calls.append(Call(layer=index_of[i]))
    plan = ModelPlan(hidden_size=hid, vocab_size=config.vocab_size, max_positions=config.max_position_embeddings,
                     embedding=EmbeddingSpec(vocab_size=config.vocab_size, hidden_size=hid, scale=config.embedding_scale),
                     layers=tuple(layers), calls=tuple(calls), final_norm=norm,
                     head=HeadSpec(vocab_size=config.vocab_size, hidden_size=hid))
    plan.validate()
    return plan


def _owners(config: ZedudraConfig):
    """Config indices of the layers that own tensors, in the plan's order."""
    return [i for i, l in enumerate(config.layers) if l.weights_of is None]


_MIXER_NAMES = {"q": "q", "k": "k", "head_gate": "g", "o": "o"}


def zedudra_tensor_name(config: ZedudraConfig, loc: TensorLocation) -> str:
    if loc.layer is None:
        if loc.role == "embedding":
            return "embed"
        if loc.role == "final_norm":
            return "final.norm"
        if loc.role == "head":
            return "head"
        raise KeyError(loc)
    prefix = f"l{_owners(config)[loc.layer]}."
    if loc.role == "mixer":
        return prefix + "mix." + _MIXER_NAMES[loc.name]
    if loc.role == "ffn":
        if "." in loc.name:                          # an expert's tensor: "gate.3" is stored as e3.gate
            what, expert = loc.name.split(".")
            return f"{prefix}mlp.e{expert}.{what}"
        return prefix + "mlp." + loc.name
    if loc.role == "block":
        return prefix + {"canon": "canon1"}[loc.name]
    if loc.role.startswith("norm."):
        return prefix + loc.role[len("norm."):]
    raise KeyError(loc)


def zedudra_ignorable(config: ZedudraConfig) -> FrozenSet[str]:
    # a layer without a feed-forward may still store the two norms around it
    return frozenset(f"l{i}.{n}" for i, l in enumerate(config.layers) if l.mlp is None and l.weights_of is None
                     for n in ("norm2", "norm2b"))


ZEDUDRA = register_architecture(Architecture(
    name=ZedudraConfig.architecture,
    config_class=ZedudraConfig,
    plan=zedudra_plan,
    tensor_name=zedudra_tensor_name,
    ignorable=zedudra_ignorable,
))
