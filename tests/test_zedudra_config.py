"""Zedudra without a GPU: configuration, errors, plan, tensor names, cache needs and retention, and the plain
model's own consistency (a sequence fed in pieces through its state gives what it gives whole)."""
import copy

import pytest
import torch

from zedudra_helpers import ZED, ZED_A, ZED_B, ZED_C, ZED_D, ZED_E, as_f64, make_weights, random_tokens, tensor_shapes
from plain import zedudra_plain as plain


def load(cfg):
    from minivllm_amd.models import config_from_dict
    return config_from_dict(copy.deepcopy(cfg))


@pytest.mark.parametrize("name", sorted(ZED))
def test_config_round_trip_and_tensor_names(name):
    from minivllm_amd.models.causal_lm import expected_tensors
    arch, cfg = load(ZED[name])
    assert arch.name == "Zedudra" and cfg.vocab_size == ZED[name]["vocab"]
    assert type(cfg).from_dict(cfg.to_dict()) == cfg
    expected = expected_tensors(arch, cfg)
    assert {k: tuple(v.shape) for k, v in expected.items()} == tensor_shapes(ZED[name])


def test_defaults_and_optional_keys():
    _, b = load(ZED_B)
    assert (b.layers[0].mlp.groups, b.layers[0].mlp.groups_keep) == (1, 1) and b.layers[0].mixer.keep_first == 0
    assert b.layers[2].weights_of == 1 and b.layers[2].mixer == b.layers[1].mixer
    _, e = load(ZED_E)
    assert e.conv_taps == 0 and e.norm_groups == 2
    _, d = load(ZED_D)
    assert d.layers[0].mixer.rot_dims == 0 and d.conv_taps == 1
    bare = copy.deepcopy(ZED_E)
    bare.pop("embedding")
    bare["norm"].pop("groups")
    bare["layers"][0]["mixer"].pop("kv_heads")
    bare["layers"][0]["mixer"].pop("vdim")
    bare["layers"][0]["mixer"].pop("scale")
    _, c = load(bare)
    assert c.embedding_scale == 1.0 and c.norm_groups == 1
    assert c.layers[0].mixer.kv_heads == 4 and c.layers[0].mixer.vdim == 12 and c.layers[0].mixer.scale == 12 ** -0.5


@pytest.mark.parametrize("edit, message", [
    (lambda c: c["layers"][0].update(type="conv"), "not supported"),
    (lambda c: c["layers"][0]["mixer"].update(kv_heads=3), "multiple"),
    (lambda c: c["layers"][0]["mixer"].update(vdim=8), "vdim"),
    (lambda c: c["layers"][0]["mixer"]["mask"].update(size=0), "mask.size"),
    (lambda c: c["layers"][0]["mixer"]["rot"].update(dims=7), "rot.dims"),
    (lambda c: c["layers"][0]["mixer"].pop("mask"), "mask"),
    (lambda c: c["layers"][1]["mlp"]["router"]["groups"].update(count=3), "groups"),
    (lambda c: c["layers"][1]["mlp"]["router"].update(top=5), "top"),
    (lambda c: c["layers"][1]["mlp"]["expert"].update(limit=0.0), "limit"),
    (lambda c: c["layers"][0]["mlp"].update(kind="sparse"), "not supported"),
    (lambda c: c["layers"][2].update(weights_of=2), "weights_of"),
    (lambda c: c["layers"][3].update(weights_of=5), "weights_of"),
    (lambda c: (c["layers"][2].update(weights_of=3), c["layers"][3].update(weights_of=2)), "weights_of"),
    (lambda c: c["layers"][3].update(weights_of=0), "other sizes"),
    (lambda c: c["layers"][2]["mixer"]["mask"].update(size=13), "other sizes"),
    (lambda c: c["norm"].update(groups=3), "norm groups"),
    (lambda c: c["canon"].update(taps=40), "canon.taps"),
    (lambda c: c.pop("norm"), "norm"),
])
def test_config_errors(edit, message):
    from minivllm_amd.config import ConfigError
    cfg = copy.deepcopy(ZED_A)
    edit(cfg)
    with pytest.raises(ConfigError, match=message):
        load(cfg)


def test_a_layer_may_name_a_later_one_or_one_that_names_another():
    from minivllm_amd.models.causal_lm import expected_tensors
    arch, want = load(ZED_A)
    chained = copy.deepcopy(ZED_A)
    chained["layers"][3]["weights_of"] = 2                      # 3 -> 2 -> 1
    _, cfg = load(chained)
    assert [c.layer for c in arch.plan(cfg).calls] == [0, 1, 1, 1, 2]
    assert set(expected_tensors(arch, cfg)) == set(expected_tensors(arch, want))
    ahead = copy.deepcopy(ZED_A)
    ahead["layers"][1]["weights_of"] = 3                        # the tensors are the fourth entry's: l3.*
    ahead["layers"][2]["weights_of"] = 3
    del ahead["layers"][3]["weights_of"]
    _, cfg = load(ahead)
    assert [c.layer for c in arch.plan(cfg).calls] == [0, 1, 1, 1, 2]
    names = set(expected_tensors(arch, cfg))
    assert "l3.mix.q" in names and not any(n.startswith(("l1.", "l2.")) for n in names)


def test_plan_parts_calls_and_memory():
    from minivllm_amd.parts.attention import Attention, AttentionSpec
    from minivllm_amd.parts.base import KeepAll, KeepWindowAndFirst, KeepWindow
    from minivllm_amd.parts.block import SandwichBlock
    from minivllm_amd.parts.mlp import XIELUSpec
    from minivllm_amd.parts.moe import RoutedExpertsSpec
    from minivllm_amd.parts.norm import GroupRMSNormSpec
    arch, cfg = load(ZED_A)
    plan = arch.plan(cfg)
    # five entries, three layers with tensors: the second runs three times, each call with a cache of its own
    assert [c.layer for c in plan.calls] == [0, 1, 1, 1, 2] and all(c.cache_from is None for c in plan.calls)
    first, second, last = plan.layers
    assert isinstance(first.ffn, XIELUSpec) and isinstance(second.ffn, RoutedExpertsSpec) and last.ffn is None
    assert (second.ffn.scoring, second.ffn.group_worth, second.ffn.normalize, second.ffn.activation, second.ffn.limit) == \
        ("sigmoid", "top2", False, "clamped", 1.5)
    m = first.mixer
    assert isinstance(m, AttentionSpec) and m.kept and not m.plain and m.value_from_key and m.head_gate
    assert m.window == 11 and m.keep_first == 5 and m.position.interleaved and m.position.rotary_dim == 8
    assert set(Attention.tensors(m)) == {"q", "k", "o", "head_gate"}
    assert all(isinstance(n, GroupRMSNormSpec) and n.groups == 4 for _, n in first.norms)
    assert [s for s, _ in last.norms] == ["norm1", "norm1b"]
    assert plan.embedding.scale == 2.5
    # the cache: keys rotated and the same keys unrotated as values; pages between the kept first ones and the window go back
    need = Attention.cache_need(m)
    assert need.page_shapes(8) == {"k": (2, 8, 16), "v": (2, 16, 8)}
    assert need.retention == KeepWindowAndFirst(11, 5)
    assert Attention.cache_need(last.mixer).retention == KeepWindow(19)
    # a request's state: the mixer's input rows of the last two tokens, in every call
    assert SandwichBlock.state_shapes(first.block) == {"conv.last": ((2, 64), None)}
    _, d = load(ZED_D)
    assert SandwichBlock.state_shapes(arch.plan(d).layers[0].block) == {}          # one tap looks at no earlier row
    _, e = load(ZED_E)
    assert SandwichBlock.state_shapes(arch.plan(e).layers[0].block) == {} and SandwichBlock.tensors(arch.plan(e).layers[0].block) == {}


def test_kept_first_pages_stay_while_the_window_moves_on():
    """The retention rule through the cache manager: pages of the kept first positions are never given back, those
    between them and the window are, and a released request returns everything."""
    from minivllm_amd.cache.manager import CacheManager, GroupSpec
    from minivllm_amd.parts.base import KeepWindowAndFirst
    rule = KeepWindowAndFirst(window=10, first=5)
    assert rule.leading_pages_kept(4) == 2 and rule.leading_pages_kept(8) == 1 and KeepWindowAndFirst(3, 0).leading_pages_kept(4) == 0
    m = CacheManager([GroupSpec(rule, (0,))], num_pages=12, page_size=4, num_state_slots=2)
    m.admit("a")
    held = []
    for step in (7, 9, 1, 1, 14, 1):
        m.reserve("a", step)
        m.commit("a", step)
        n = m.sequence("a").num_computed
        table = m.block_table("a", 0)
        first_needed = max(0, n - 10) // 4
        for i, p in enumerate(table):
            assert (p >= 0) == (i < 2 or i >= first_needed), (n, i, table)
        held.append(sum(p >= 0 for p in table))
        m.check_invariants()
    assert max(held) <= rule.most_pages_held(33, 4, 14)
    m.release("a")
    assert m.num_free_pages(0) == 12


@pytest.mark.parametrize("name", sorted(ZED))
def test_plain_model_in_pieces_is_the_plain_model_whole(name):
    cfg = ZED[name]
    w = as_f64(make_weights(cfg, seed=5))
    toks = random_tokens(cfg, 45, seed=3)
    whole, _ = plain.forward(cfg, w, toks)
    state, rows, p = None, [], 0
    for n in (1, 2, 1, 7, 3, 30, 1):
        logits, state = plain.forward(cfg, w, toks[p:p + n], start=p, state=state)
        rows.append(logits)
        p += n
    assert torch.allclose(torch.cat(rows), whole, atol=1e-10)


def test_plain_visibility_and_router_properties():
    assert plain.visible(50, 50, 1, 0) and not plain.visible(50, 49, 1, 0) and not plain.visible(3, 4, 9, 9)
    assert plain.visible(50, 41, 10, 0) and not plain.visible(50, 40, 10, 0)
    assert plain.visible(50, 4, 10, 5) and not plain.visible(50, 5, 10, 5)
    v = plain.visibility(3, 4, 2, 1)
    assert v.tolist() == [[plain.visible(i, j, 2, 1) for j in range(7)] for i in range(3, 7)]
    # a group is worth its two best: group 1 (0.9 + 0.1) loses to group 0 (0.6 + 0.55) although it holds the best expert
    z = torch.logit(torch.tensor([[0.6, 0.55, 0.2, 0.9, 0.1, 0.05]], dtype=torch.float64))
    ids, weights = plain.route(z, groups=2, keep=1, top=2)
    assert ids[0].tolist() == [0, 1] and torch.allclose(weights, torch.tensor([[0.6, 0.55]], dtype=torch.float64))
    ids, weights = plain.route(z, groups=2, keep=2, top=2)                 # every group kept: the two best overall
    assert ids[0].tolist() == [3, 0]
    assert torch.allclose(weights.sum(), torch.tensor(1.5, dtype=torch.float64))    # not renormalised
    ids, _ = plain.route(z, groups=6, keep=2, top=2)                       # groups of one: worth their one score
    assert ids[0].tolist() == [3, 0]


def test_plain_convolution_and_activation_edges():
    taps = torch.tensor([[0.5, -1.0, 2.0]], dtype=torch.float64)            # one channel, three taps
    h = torch.tensor([[1.0], [10.0], [100.0]], dtype=torch.float64)
    y, last = plain.input_conv(h, taps)
    assert y[:, 0].tolist() == [1 + 2.0, 10 - 1 + 20, 100 + 0.5 - 10 + 200] and last[:, 0].tolist() == [10.0, 100.0]
    y2, _ = plain.input_conv(h[2:], taps, before=h[:2])
    assert y2[0, 0] == y[2, 0]
    z = torch.tensor([-3.0, 0.0, 2.0], dtype=torch.float64)
    p, q = torch.tensor(0.3, dtype=torch.float64), torch.tensor(-0.4, dtype=torch.float64)
    a = plain.xielu(z, p, q)
    sp = lambda t: torch.log1p(torch.exp(t))
    assert torch.allclose(a[2], sp(p) * 4 + 1) and a[1] == 0
    assert torch.allclose(a[0], (0.5 + sp(q)) * (torch.exp(z[0]) - 1 - z[0]) + z[0] / 2)
    g = plain.grouped_rms_norm(torch.tensor([[3.0, 4.0, 0.0, 2.0]], dtype=torch.float64), torch.ones(4, dtype=torch.float64), 2, 0.0)
    assert torch.allclose(g, torch.tensor([[3 / 12.5 ** 0.5, 4 / 12.5 ** 0.5, 0.0, 2 ** 0.5]], dtype=torch.float64))
