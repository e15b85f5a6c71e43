"""Furanex on the CPU: the configuration's round trip, defaults and errors, the plan and what it asks of the cache, the
stretched rotation frequencies, and the plain model whole against in pieces."""
import copy
import math

import numpy as np
import pytest
import torch

from furanex_helpers import FUR, make_weights, plain_logits, random_config, random_tokens, tensor_shapes
from plain import furanex_plain as plain

from minivllm_amd.config.model_config import ConfigError, FuranexConfig
from minivllm_amd.models import config_from_dict, expected_tensors


@pytest.mark.parametrize("name", sorted(FUR))
def test_round_trip_and_tensor_names(name):
    arch, cfg = config_from_dict(FUR[name])
    assert arch.name == "Furanex" and isinstance(cfg, FuranexConfig)
    assert FuranexConfig.from_dict(cfg.to_dict()) == cfg
    expected, stored, spare = expected_tensors(arch, cfg), tensor_shapes(FUR[name]), arch.ignorable(cfg)
    assert set(expected) | {n for n in stored if n in spare} == set(stored)
    assert all(tuple(expected[n].shape) == tuple(stored[n]) for n in expected)
    # the head is the embedding's table, and the first value-sharing layer's blend weight is stored but unused
    assert "head" not in expected and all(n.endswith(".vmix") for n in spare if n in stored)


def test_configurations_drawn_at_random_parse():
    for seed in range(20):
        raw = random_config(np.random.default_rng(seed), fast_sizes=seed % 2 == 0)
        arch, cfg = config_from_dict(raw)
        assert set(expected_tensors(arch, cfg)) <= set(tensor_shapes(raw))


def test_defaults():
    raw = copy.deepcopy(FUR["E"])
    del raw["embedding"]
    m = raw["layers"][0]["mixer"]
    del m["kv_heads"], m["vdim"], m["scale"], m["v_mix"], m["rot"]["scaling"]
    raw["layers"][1]["mixer"]["v_mix"] = False
    cfg = FuranexConfig.from_dict(raw).completed()
    l0 = cfg.layers[0].mixer
    assert cfg.embedding_scale == 1.0 and cfg.streams == 0 and l0.kv_heads == l0.heads and l0.vdim == l0.dim
    assert l0.scale == l0.dim ** -0.5 and not l0.v_mix and l0.rot.stretch is None and cfg.first_mixing_layer() is None
    assert cfg.layers[0].mlp.shared_ff == 0 and cfg.layers[1].mlp.shared_ff == 12


@pytest.mark.parametrize("name", sorted(FUR))
def test_sizes_left_out_are_read_from_the_stored_shapes(name):
    """Everything a stored tensor's shape states may be left out of config.json: the completed configuration is the one
    that states it all. What no shape states (a head's size when the head count is left out too) is an error."""
    full = FuranexConfig.from_dict(FUR[name]).completed()
    raw = copy.deepcopy(FUR[name])
    for key in ("vocab", "width", "streams"):
        raw.pop(key, None)
    for layer in raw["layers"]:
        m = layer["mixer"]
        for key in ("heads", "kv_heads", "vdim", "q_rank", "kv_rank", "rot_dim"):
            m.pop(key, None)
        if layer["type"] == "latent_attention":
            m.pop("dim")
        if layer.get("mlp"):
            layer["mlp"].pop("shared", None)
            layer["mlp"]["expert"].pop("ff")
            layer["mlp"]["router"] = {}
    shapes = tensor_shapes(FUR[name])
    thin = FuranexConfig.from_dict(raw)
    assert thin.vocab_size == -1 and thin.layers[0].mixer.heads == -1
    assert thin.completed(lambda n: shapes.get(n)) == full
    with pytest.raises(ConfigError):
        thin.completed()
    attn = next(l for l in raw["layers"] if l["type"] == "attention")
    del attn["mixer"]["dim"]
    with pytest.raises(ConfigError):
        FuranexConfig.from_dict(raw).completed(lambda n: shapes.get(n))


def _broken(name, edit):
    raw = copy.deepcopy(FUR[name])
    edit(raw)
    return raw


@pytest.mark.parametrize("name, edit", [
    ("A", lambda c: c["layers"][0].update(type="recurrent")),
    ("A", lambda c: c["layers"][0]["mixer"].update(kv_heads=3)),
    ("A", lambda c: c["layers"][0]["mixer"]["rot"].update(dims=18)),
    ("A", lambda c: c["layers"][0]["mixer"]["rot"].update(dims=5)),
    ("A", lambda c: c["layers"][2]["mixer"].update(vdim=16)),                 # shares values of another size than layer 0's
    ("A", lambda c: c["layers"][1]["mixer"].update(rot_dim=6)),               # the rotated part and rot.dims disagree
    ("A", lambda c: c["layers"][0]["mlp"]["router"].update(top=6)),
    ("A", lambda c: c["layers"][0]["mlp"].update(kind="dense")),
    ("A", lambda c: c["layers"][0]["mixer"]["rot"]["scaling"].update(factor=0.0)),
    ("A", lambda c: c.update(streams=9)),
    ("A", lambda c: c["norm"].update(eps=0.0)),
    ("A", lambda c: c.pop("vocab")),
    ("B", lambda c: c["layers"][0]["mixer"].pop("kv_rank")),
])
def test_configuration_errors(name, edit):
    with pytest.raises(ConfigError):
        FuranexConfig.from_dict(_broken(name, edit)).completed()


def test_plan_and_memory():
    from minivllm_amd.parts.base import MIXERS
    arch, cfg = config_from_dict(FUR["A"])
    plan = arch.plan(cfg)
    kinds = [l.mixer.kind for l in plan.layers]
    assert kinds == ["attention", "latent_attention", "attention"] and all(l.block.kind == "hyper_connections" for l in plan.layers)
    a0, lat, a2 = (l.mixer for l in plan.layers)
    assert (a0.value_mix, a2.value_mix) == ("source", "blend") and a0.value_mix_key == a2.value_mix_key
    assert a0.unit_norm_after_rotation and a0.position.stretch == (3.0, 64.0, 16.0, 2.0) and not a0.position.interleaved
    assert lat.head_gate and lat.rot_neighbours and plan.layers[1].ffn is None and not plan.layers[1].block.has_ffn
    need = MIXERS.get(a0.kind).cache_need(a0)
    assert need.page_shapes(16) == {"k": (2, 16, 16), "v": (2, 8, 16)} and need.retention.keeps_everything
    need = MIXERS.get(lat.kind).cache_need(lat)
    assert need.page_shapes(8)["latent"] == (8, 16 + 4)
    assert plan.layers[0].ffn.router == "table" and plan.layers[0].ffn.table_rows == 200 and plan.layers[0].ffn.shared_size == 40
    # without streams the layers are plain pre-norm blocks
    arch, cfg = config_from_dict(FUR["E"])
    assert all(l.block.kind == "pre_norm" for l in arch.plan(cfg).layers)


@pytest.mark.parametrize("dims, base, stretch", [(12, 5000.0, (3.0, 64, 16.0, 2.0)), (64, 5e5, (8.0, 2048, 16.0, 2.0)),
                                                 (48, 2e4, (4.0, 256, 16.0, 1.0)), (8, 200.0, (2.0, 4000, 1000.0, 0.001)),
                                                 (4, 300.0, (8.0, 16, 4.0, 0.5)), (128, 1e6, (40.0, 4096, 32.0, 1.0))])
def test_stretched_frequencies(dims, base, stretch):
    from minivllm_amd.parts.rope import stretched_frequencies
    freqs, magnitude = stretched_frequencies(dims, base, stretch)
    want, factor = plain.rotation_frequencies(dims, base, dict(zip(("factor", "original", "fast", "slow"), stretch)))
    assert freqs.dtype == torch.float32 and np.allclose(freqs.double().numpy(), want, rtol=1e-7, atol=0)
    assert abs(magnitude - factor) < 1e-12 and abs(factor - (0.1 * math.log(stretch[0]) + 1.0)) < 1e-12
    plain_f = [base ** (-2.0 * i / dims) for i in range(dims // 2)]
    # every pair turns no faster than plainly and no slower than plainly / factor; the fastest pair is left alone when
    # the ramp starts behind it
    assert all(p / stretch[0] * (1 - 1e-12) <= f <= p * (1 + 1e-12) for f, p in zip(want, plain_f))


def test_rotation_pairs_of_the_plain_model():
    x = torch.randn(5, 2, 10, dtype=torch.float64)
    pos = torch.arange(3, 8)
    freqs, factor = plain.rotation_frequencies(6, 100.0, None)
    for neighbours in (False, True):
        y = plain.rotate(x, pos, 6, freqs, 1.0, neighbours)
        assert torch.equal(y[..., 6:], x[..., 6:])                          # channels behind the rotated ones pass
        assert torch.allclose(y[..., :6].pow(2).sum(-1), x[..., :6].pow(2).sum(-1))
        back = plain.rotate(y, -pos, 6, freqs, 1.0, neighbours)
        assert torch.allclose(back, x)
    # position 0 is the identity; a magnitude multiplies the rotated channels only
    assert torch.equal(plain.rotate(x, torch.zeros(5, dtype=torch.long), 6, freqs, 1.0, False), x)
    z = plain.rotate(x, torch.zeros(5, dtype=torch.long), 6, freqs, 1.5, True)
    assert torch.allclose(z[..., :6], 1.5 * x[..., :6]) and torch.equal(z[..., 6:], x[..., 6:])


@pytest.mark.parametrize("name", sorted(FUR))
def test_plain_model_in_pieces_is_the_whole(name):
    cfg = FUR[name]
    w = {k: (v.double() if v.is_floating_point() else v) for k, v in make_weights(cfg, seed=3).items()}
    toks = random_tokens(cfg, 41, seed=4)
    whole = plain.forward(cfg, w, toks)[0]
    rows, past, at = [], None, 0
    for k in (5, 1, 2, 13, 1, 19):
        out, past = plain.forward(cfg, w, toks[at:at + k], start=at, past=past)
        rows.append(out)
        at += k
    assert torch.allclose(torch.cat(rows), whole, rtol=1e-9, atol=1e-9)


def test_streams_of_the_plain_model():
    """With the identity as the mixing matrix, reads of 1/S and writes of 1, S streams are one plain residual."""
    xs = torch.randn(1, 4, 6, dtype=torch.float64).repeat(3, 1, 1)
    y = torch.randn(4, 6, dtype=torch.float64)
    new = plain.streams_write(xs, y, torch.eye(3), torch.ones(3))
    assert torch.allclose(new, xs + y[None]) and torch.allclose(plain.streams_read(new, torch.full((3,), 1 / 3)), xs[0] + y)
    # the mixing matrix is indexed [from, to]
    mix = torch.zeros(3, 3)
    mix[0, 2] = 1.0
    moved = plain.streams_write(torch.arange(3.0).view(3, 1, 1) + 1, torch.zeros(1, 1), mix, torch.zeros(3))
    assert moved.view(3).tolist() == [0.0, 0.0, 1.0]


def test_table_mixture_of_the_plain_model():
    cfg = FUR["A"]
    w = {k: (v.double() if v.is_floating_point() else v) for k, v in make_weights(cfg, seed=8).items()}
    f = cfg["layers"][0]["mlp"]
    h = torch.randn(3, cfg["width"], dtype=torch.float64)
    ids = torch.tensor([7, 7, 100])
    y = plain.table_mixture(h, ids, w, "l0.mlp.", f)
    e0, e1 = w["l0.mlp.table"][7].tolist()
    by_hand = (plain.expert(h[:1], w, f"l0.mlp.e{e0}.") + plain.expert(h[:1], w, f"l0.mlp.e{e1}.")) / 2 + plain.expert(h[:1], w, "l0.mlp.shared.")
    assert torch.allclose(y[:1], by_hand) and e0 != e1
