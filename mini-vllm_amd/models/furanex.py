"""Furanex as a plan of parts.

Every layer is a block on several residual streams (``parts/block.py: HyperConnectionBlock``; a plain pre-norm block
when the configuration names no streams). Its mixer is grouped softmax attention whose q and k are rotated over their
first channels in half-split pairs and then divided by their root mean square per head, whose values may have another
size than its keys and are blended, from the second such layer on, with the values the first such layer projected for
the same token (``parts/attention.py``), or attention over a cached latent with the rotated part paired by neighbours and
one output gate a head (``parts/latent_attention.py``). The rotation's low frequencies may be stretched
(``parts/rope.py: stretched_frequencies``). The feed-forward is a mixture whose experts a stored table names by token
id, each with the weight 1 / top, beside a shared expert (``parts/moe.py``); a layer may have none. The embedding is
multiplied by a constant and its table is the output head.

Tensor names on disk: ``embed``, ``final.norm``; per layer i ``l<i>.norm1``, ``.norm2``, ``l<i>.hc<q>.{in,out,mix}``,
``l<i>.mix.{q,k,v,vmix,o}`` or ``l<i>.mix.{dq,dq.norm,uq,dkv,dkv.norm,uk,uv,g,o}``, ``l<i>.mlp.{table,e<j>.gate|up|down,
shared.gate|up|down}``.
"""
from __future__ import annotations

from typing import FrozenSet

from ..config.model_config import FuranexConfig
from ..parts.attention import AttentionSpec
from ..parts.block import HyperConnectionBlock, HyperConnectionBlockSpec, PreNormBlock, PreNormBlockSpec
from ..parts.latent_attention import LatentAttentionSpec
from ..parts.moe import RoutedExpertsSpec
from ..parts.norm import RMSNormSpec
from ..parts.plan import Call, EmbeddingSpec, HeadSpec, LayerPlan, ModelPlan, TensorLocation
from ..parts.rope import RotarySpec
from .registry import Architecture, register_architecture

VALUE_MIX_KEY = "values.first"     # where the first value-sharing layer leaves its values for the step's later layers


def furanex_plan(config: FuranexConfig) -> ModelPlan:
    # (sizes that config.json left out and no loader has filled in from the stored tensors take their defaults here,
    # or are an error when they have none)
    config = config.completed()
    hid = config.hidden_size
    norm = RMSNormSpec(size=hid, eps=config.norm_eps)
    first_mix = config.first_mixing_layer()
    layers = []
    for i, l in enumerate(config.layers):
        m = l.mixer
        if m.kind == "attention":
            rope = None if m.rot is None else RotarySpec(rotary_dim=m.rot.dims, theta=m.rot.base, interleaved=False,
                                                         stretch=m.rot.stretch)
            mix = None if not m.v_mix else ("source" if i == first_mix else "blend")
            mixer = AttentionSpec(hidden_size=hid, num_heads=m.heads, num_kv_heads=m.kv_heads, head_dim=m.dim, scale=m.scale,
                                  qk_norm=False, qk_norm_eps=config.norm_eps, bias=False, window=None, position=rope,
                                  value_dim=m.vdim, unit_norm_after_rotation=True, value_mix=mix,
                                  value_mix_key=VALUE_MIX_KEY if mix else "")
        else:
            # the part rotates in half-split pairs over rows it has put in that order itself (``rot_neighbours``)
            rope = None if not m.rot_dim else RotarySpec(rotary_dim=m.rot_dim, theta=m.rot.base, interleaved=False,
                                                         stretch=m.rot.stretch)
            mixer = LatentAttentionSpec(hidden_size=hid, num_heads=m.heads, plain_dim=m.dim, rot_dim=m.rot_dim, value_dim=m.vdim,
                                        q_rank=m.q_rank, kv_rank=m.kv_rank, scale=m.scale, norm_eps=config.norm_eps,
                                        output_gate=True, head_gate=True, rot_neighbours=True, position=rope)
        f = l.mlp
        ffn = None
        if f is not None:
            ffn = RoutedExpertsSpec(hidden_size=hid, expert_size=f.ff, num_experts=f.experts, top=f.top, router="table",
                                    table_rows=config.vocab_size, shared_size=f.shared_ff)
        if config.streams:
            block = HyperConnectionBlockSpec(hidden_size=hid, streams=config.streams, has_ffn=ffn is not None)
            slots = HyperConnectionBlock.slots_for(ffn is not None)
        else:
            block = PreNormBlockSpec()
            slots = PreNormBlock.slots_for(ffn is not None)
        layers.append(LayerPlan(block=block, mixer=mixer, ffn=ffn, norms=tuple((s, norm) for s in slots)))
    plan = ModelPlan(hidden_size=hid, vocab_size=config.vocab_size, max_positions=config.max_position_embeddings,
                     embedding=EmbeddingSpec(vocab_size=config.vocab_size, hidden_size=hid, scale=config.embedding_scale),
                     layers=tuple(layers), calls=tuple(Call(layer=i) for i in range(len(layers))), final_norm=norm,
                     head=HeadSpec(vocab_size=config.vocab_size, hidden_size=hid, tied=True))
    plan.validate()
    return plan


_ATTENTION_NAMES = {"q": "q", "k": "k", "v": "v", "o": "o", "value_mix": "vmix"}
_LATENT_NAMES = {"dq": "dq", "dq_norm": "dq.norm", "uq": "uq", "dkv": "dkv", "dkv_norm": "dkv.norm", "uk": "uk", "uv": "uv",
                 "g": "g", "o": "o"}
_NORM_SLOTS = {"mixer": "norm1", "ffn": "norm2", "norm1": "norm1", "norm2": "norm2"}


def furanex_tensor_name(config: FuranexConfig, loc: TensorLocation) -> str:
    if loc.layer is None:
        if loc.role in ("embedding", "head"):
            return "embed"                               # the head is the embedding's table
        if loc.role == "final_norm":
            return "final.norm"
        raise KeyError(loc)
    prefix = f"l{loc.layer}."
    if loc.role == "mixer":
        names = _ATTENTION_NAMES if config.layers[loc.layer].mixer.kind == "attention" else _LATENT_NAMES
        return prefix + "mix." + names[loc.name]
    if loc.role == "ffn":
        parts = loc.name.split(".")
        if len(parts) == 2 and parts[1].isdigit():       # an expert's tensor: "gate.3" is stored as e3.gate
            return f"{prefix}mlp.e{parts[1]}.{parts[0]}"
        return prefix + "mlp." + loc.name                # table, shared.gate, ...
    if loc.role == "block":
        return prefix + loc.name                         # hc1.in, hc2.mix, ...
    if loc.role.startswith("norm."):
        return prefix + _NORM_SLOTS[loc.role[len("norm."):]]
    raise KeyError(loc)


def furanex_complete(config: FuranexConfig, source) -> FuranexConfig:
    """The configuration with what only the stored tensors state, where config.json leaves it out: vocabulary and width
    are the embedding's shape, the streams the length of ``l0.hc1.in``, head counts and sizes the rows of the projections,
    the ranks the lengths of the latent norms, the rotated channels what ``dkv`` has beyond the latent, an expert's width
    the rows of ``e0.gate``, the experts their number, ``top`` the table's columns, a shared expert's width the rows of
    ``shared.gate`` (none when there is no such tensor)."""
    names = set(source.names())
    return config.completed(lambda name: tuple(source.shape(name)) if name in names else None)


def furanex_ignorable(config: FuranexConfig) -> FrozenSet[str]:
    # the first value-sharing layer stores a blend weight it never uses; a layer without a feed-forward may still
    # store the norm and the stream weights in front of it
    first = config.first_mixing_layer()
    names = set() if first is None else {f"l{first}.mix.vmix"}
    for i, l in enumerate(config.layers):
        if l.mlp is None:
            names.update(f"l{i}.{n}" for n in ("norm2", "hc2.in", "hc2.out", "hc2.mix"))
    return frozenset(names)


FURANEX = register_architecture(Architecture(
    name=FuranexConfig.architecture,
    config_class=FuranexConfig,
    plan=furanex_plan,
    tensor_name=furanex_tensor_name,
    ignorable=furanex_ignorable,
    complete=furanex_complete,
))
