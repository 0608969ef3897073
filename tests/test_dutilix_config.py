"""Dutilix without a GPU: configuration, errors, plan, tensor names, cache needs, and the plain model's own
consistency (a sequence fed in pieces through its states gives what it gives whole)."""
import copy

import pytest
import torch

from dutilix_helpers import DUT, DUT_A, DUT_B, DUT_D, as_f64, make_weights, random_tokens, tensor_shapes
from plain import dutilix_plain as plain


def load(cfg):
    from minivllm_amd.models import config_from_dict
    return config_from_dict(copy.deepcopy(cfg))


@pytest.mark.parametrize("name", sorted(DUT))
def test_config_round_trip_and_tensor_names(name):
    from minivllm_amd.models.causal_lm import expected_tensors
    arch, cfg = load(DUT[name])
    assert arch.name == "Dutilix" and cfg.vocab_size == DUT[name]["vocab"]
    again = type(cfg).from_dict(cfg.to_dict())
    assert again == cfg
    expected = expected_tensors(arch, cfg)
    assert {k: tuple(v.shape) for k, v in expected.items()} == tensor_shapes(DUT[name])


def test_defaults_and_optional_keys():
    _, cfg = load(DUT_B)
    assert cfg.logit_scale == 1.0
    first, third = cfg.layers[0].mlp, cfg.layers[2].mlp
    assert (first.groups, first.groups_keep, first.identity) == (1, 1, 0)
    assert (third.groups, third.groups_keep, third.identity, third.experts) == (3, 2, 3, 3)
    assert cfg.layers[3].mlp is None and cfg.layers[3].mixer.kv_heads == 1
    _, d = load(DUT_D)
    assert d.layers[1].mixer.rot_dim == 0 and d.layers[0].mixer.conv == 1


@pytest.mark.parametrize("edit, message", [
    (lambda c: c["layers"][0].update(type="conv"), "not supported"),
    (lambda c: c["layers"][0]["mixer"].update(kv_heads=3), "multiple"),
    (lambda c: c["layers"][0]["mixer"].update(conv=-2), "conv"),
    (lambda c: c["layers"][0]["mlp"]["router"]["groups"].update(count=4), "groups"),
    (lambda c: c["layers"][0]["mlp"]["router"].update(top=7), "top"),
    (lambda c: c["layers"][1]["mixer"]["rot"].update(dims=4), "rot.dims"),
    (lambda c: c["layers"][1]["mixer"].update(rot_dim=7), "rot"),
    (lambda c: c["layers"][2]["mixer"].update(gate_cap=0.0), "gate_cap"),
    (lambda c: c["layers"][1]["mlp"].update(kind="sparse"), "not supported"),
    (lambda c: c.pop("norm"), "norm"),
])
def test_config_errors(edit, message):
    from minivllm_amd.config import ConfigError
    cfg = copy.deepcopy(DUT_A)
    edit(cfg)
    with pytest.raises(ConfigError, match=message):
        load(cfg)


def test_plan_parts_and_memory():
    from minivllm_amd.parts import GatedDeltaSpec, LatentAttentionSpec, MLSTMSpec, RoutedExpertsSpec, ScaledHeadSpec, SwiGLUSpec
    from minivllm_amd.parts.base import MIXERS, KeepAll
    arch, cfg = load(DUT_A)
    plan = arch.plan(cfg)
    kinds = [type(l.mixer) for l in plan.layers]
    assert kinds == [GatedDeltaSpec, LatentAttentionSpec, MLSTMSpec, LatentAttentionSpec]
    assert [type(l.ffn) for l in plan.layers] == [RoutedExpertsSpec, SwiGLUSpec, type(None), RoutedExpertsSpec]
    assert [len(l.norms) for l in plan.layers] == [2, 2, 1, 2]
    assert isinstance(plan.head, ScaledHeadSpec) and plan.head.scale == 0.5
    d, la, ml = plan.layers[0].mixer, plan.layers[1].mixer, plan.layers[2].mixer
    assert (d.num_heads, d.num_kv_heads, d.key_dim, d.value_dim, d.conv_taps) == (4, 2, 16, 24, 4)
    states = MIXERS.get(d.kind).state_shapes(d)
    assert states["state"] == ((4, 24, 16), torch.float32) and states["conv"][0] == (3, 2 * 2 * 16 + 4 * 24)
    assert MIXERS.get(ml.kind).state_shapes(ml) == {"state": ((2, 21, 16), torch.float32), "max": ((2,), torch.float32)}
    need = MIXERS.get(la.kind).cache_need(la)
    assert need.page_shapes(8) == {"latent": (8, 32 + 8), "latent_t": (32, 8)} and isinstance(need.retention, KeepAll)
    assert need.bytes_per_token(torch.bfloat16) == 80 + 64 and MIXERS.get(d.kind).cache_need(d) is None
    r = plan.layers[0].ffn
    assert (r.num_experts, r.identity_experts, r.top, r.groups, r.keep_groups, r.router_outputs) == (8, 2, 3, 5, 3, 10)
    # the two attention layers keep everything: one cache group
    assert len({MIXERS.get(l.mixer.kind).cache_need(l.mixer).group_key() for l in plan.layers if l.mixer.kind == "latent_attention"}) == 1


def test_a_single_tap_needs_no_convolution_state():
    from minivllm_amd.parts.base import MIXERS
    arch, cfg = load(DUT_D)
    spec = arch.plan(cfg).layers[0].mixer
    assert set(MIXERS.get(spec.kind).state_shapes(spec)) == {"state"}


@pytest.mark.parametrize("name", ["A", "B", "D"])
def test_plain_model_in_pieces_is_the_plain_model_whole(name):
    cfg = DUT[name]
    w = as_f64(make_weights(cfg, seed=5))
    toks = random_tokens(cfg, 37, seed=2)
    whole, _ = plain.forward(cfg, w, toks)
    states, rows = None, []
    for lo, hi in ((0, 1), (1, 3), (3, 20), (20, 21), (21, 37)):
        part, states = plain.forward(cfg, w, toks[lo:hi], states)
        rows.append(part)
    assert float((torch.cat(rows) - whole).abs().max() / whole.abs().max()) < 1e-10


def test_plain_router_properties():
    g = torch.Generator().manual_seed(0)
    h = torch.randn(50, 16, generator=g, dtype=torch.float64)
    router = torch.randn(12, 16, generator=g, dtype=torch.float64)
    correction = torch.randn(12, generator=g, dtype=torch.float64)
    chosen, weight = plain.route(h, router, correction, top=3, groups=4, keep=2)
    assert chosen.shape == (50, 3) and torch.allclose(weight.sum(-1), torch.ones(50, dtype=torch.float64))
    assert all(len({int(e) // 3 for e in row}) <= 2 and len(set(row.tolist())) == 3 for row in chosen)
    # the correction moves the choice, not the weights: the weights are the plain scores, renormalised
    score = torch.softmax(h @ router.T, -1)
    picked = score.gather(1, chosen)
    assert torch.allclose(weight, picked / picked.sum(-1, keepdim=True))
    free, _ = plain.route(h, router, torch.zeros(12, dtype=torch.float64), top=3, groups=1, keep=1)
    assert (free != chosen).any()
    assert torch.equal(free.sort(-1).values, score.topk(3, -1).indices.sort(-1).values)


def test_plain_short_convolution_edges():
    x = torch.arange(12, dtype=torch.float64).view(6, 2) + 1
    taps = torch.tensor([[1.0, 10.0, 100.0], [0.0, 0.0, 1.0]], dtype=torch.float64)
    y, kept = plain.short_conv(x, taps)
    assert y[0].tolist() == [100.0, 2.0] and y[2].tolist() == [100 * 5 + 10 * 3 + 1, 6.0]
    assert torch.equal(kept, x[-2:])
    y2, kept2 = plain.short_conv(x[4:], taps, before=plain.short_conv(x[:4], taps)[1])
    assert torch.equal(y2, y[4:]) and torch.equal(kept2, kept)
    y1, kept1 = plain.short_conv(x[:1], taps)
    assert torch.equal(kept1, torch.stack([torch.zeros(2, dtype=torch.float64), x[0]]))


def test_sizes_that_config_json_leaves_out_come_from_the_tensors():
    """Taps, both ranks and the attention's scale may be absent: taps and ranks are read off the stored tensors'
    shapes, the scale is (dim + rot_dim)^-1/2."""
    from minivllm_amd.weights.source import DictSource
    cfg = copy.deepcopy(DUT_A)
    del cfg["layers"][0]["mixer"]["conv"]
    for key in ("q_rank", "kv_rank", "scale"):
        del cfg["layers"][1]["mixer"][key]
    arch, bare = load(cfg)
    with pytest.raises(ValueError, match="taps"):
        arch.plan(bare)
    weights = make_weights(DUT_A, seed=1)
    full = arch.complete(bare, DictSource(weights))
    _, want = load(DUT_A)
    assert full.layers[0] == want.layers[0] and full.layers[2:] == want.layers[2:]
    got, ref = full.layers[1].mixer, want.layers[1].mixer
    assert (got.q_rank, got.kv_rank) == (ref.q_rank, ref.kv_rank) and abs(got.scale - (16 + 8) ** -0.5) < 1e-12
    arch.plan(full)
