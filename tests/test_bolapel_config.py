"""Bolapel on the CPU: configuration, plan, tensor names, retention by chunks, the cache manager with
it, and the plain model's own consistency (a state carried over a cut gives what the whole gives)."""
import copy
import json
import os

import numpy as np
import pytest
import torch

from bolapel_helpers import BOLA, RANKS, make_weights, tensor_shapes
from plain import bolapel_plain as plain

from minivllm_amd.cache.manager import CacheManager, GroupSpec, groups_from_needs
from minivllm_amd.config import BolapelConfig, ConfigError
from minivllm_amd.models import config_from_dict, get_architecture
from minivllm_amd.models.causal_lm import expected_tensors
from minivllm_amd.parts import MIXERS, KeepAll, KeepChunks
from minivllm_amd.weights.source import DictSource


def completed(name):
    arch, cfg = config_from_dict(copy.deepcopy(BOLA[name]))
    weights = make_weights(BOLA[name], RANKS[name], seed=1)
    return arch, arch.complete(cfg, DictSource(weights)), weights


@pytest.mark.parametrize("name", sorted(BOLA))
def test_expected_tensors_are_the_folder(name):
    arch, cfg, weights = completed(name)
    expected = expected_tensors(arch, cfg)
    assert {k: tuple(v.shape) for k, v in expected.items()} == tensor_shapes(BOLA[name], RANKS[name])
    assert all(l.decay_rank == RANKS[name] for l in cfg.layers if l.type == "general_delta")


@pytest.mark.parametrize("name", sorted(BOLA))
def test_config_round_trip(name):
    arch, cfg, _ = completed(name)
    again = BolapelConfig.from_dict(json.loads(json.dumps(cfg.to_dict())))
    assert again == cfg
    assert arch is get_architecture("Bolapel")


def test_plan_of_Q():
    arch, cfg, _ = completed("Q")
    plan = arch.plan(cfg)
    assert [c.cache_from for c in plan.calls] == [None, None, None, None, 2]
    needs = [None if l.mixer is None else MIXERS.get(l.mixer.kind).cache_need(l.mixer) for l in plan.layers]
    assert needs[1] is None and needs[3] is None and needs[4] is None
    # the owner keeps a page while the reader's larger chunk still needs it
    assert needs[0].retention == KeepChunks((7,)) and needs[2].retention == KeepChunks((33, 50))
    assert needs[2].page_shapes(8) == {"k": (1, 8, 64), "v": (1, 40, 8)}
    groups = groups_from_needs(needs)
    assert [g.calls for g in groups] == [(0,), (2,)]
    assert plan.layers[2].ffn is None and [s for s, _ in plan.layers[2].norms] == ["norm1", "norm1b"]
    assert plan.head.kind == "linear_head"
    plan_p = completed("P")[0].plan(completed("P")[1])
    assert plan_p.head.kind == "capped_linear_head" and plan_p.head.cap == 12.0
    s = completed("S")[0].plan(completed("S")[1]).layers[0].mixer
    assert isinstance(MIXERS.get(s.kind).cache_need(s).retention, KeepAll) and s.position is None


@pytest.mark.parametrize("edit, message", [
    (lambda c: c["layers"][1]["mixer"].update(kv_from=3), "kv_from"),
    (lambda c: c["layers"][3]["mixer"].update(kv_from=0), "kv_from"),
    (lambda c: c["layers"][3]["mixer"].update(dim=16), "kv_from"),
    (lambda c: c["layers"][1]["mixer"].update(kv_heads=3), "multiple"),
    (lambda c: c["layers"][1]["mixer"]["rot"].update(dims=34), "rot.dims"),
    (lambda c: c["layers"][1]["mixer"]["mask"].update(size=0), "mask.size"),
    (lambda c: c["layers"][0].update(type="conv"), "not supported"),
    (lambda c: c["layers"][0]["mlp"].update(kind="routed"), "dense"),
    (lambda c: c.pop("norm"), "norm"),
    (lambda c: c.update(logit_softcap=-1.0), "logit_softcap"),
    (lambda c: c["layers"][1]["mixer"].pop("scale"), "scale"),
])
def test_config_errors(edit, message):
    cfg = copy.deepcopy(BOLA["P"])
    edit(cfg)
    with pytest.raises(ConfigError, match=message):
        config_from_dict(cfg)


def test_keep_chunks():
    rule = KeepChunks((20,))
    assert [rule.first_kept_page(p, 8) for p in (0, 19, 20, 39, 40, 47, 48)] == [0, 0, 2, 2, 5, 5, 5]
    both = KeepChunks((20, 30))
    for p in range(0, 200):
        assert both.first_kept_page(p, 4) == min(p // 20 * 20, p // 30 * 30) // 4
    assert list(both.first_kept_pages(np.arange(0, 200), 4)) == [both.first_kept_page(p, 4) for p in range(200)]
    assert KeepChunks((20,)).key() != KeepChunks((20, 30)).key() and not rule.keeps_everything
    with pytest.raises(ValueError):
        KeepChunks(())


def test_manager_gives_back_pages_a_chunk_has_passed():
    m = CacheManager([GroupSpec(KeepChunks((20,)), (0,))], 8, 4, 2, has_state=True)
    assert not m.prefix_caching
    m.admit("a")
    done = 0
    for n in (7, 13, 1, 1, 30, 3):
        m.reserve("a", n)
        m.commit("a", n)
        done += n
        table = m.block_table("a", 0)
        first = done // 20 * 20 // 4
        assert all(p < 0 for p in table[:first]) and all(p >= 0 for p in table[first:])
        m.check_invariants()
    m.release("a")
    assert m.pools[0].num_free == 8 and m.slots.num_free == 2


def test_plain_state_carry_equals_whole():
    g = torch.Generator().manual_seed(3)
    n, dk, dv = 23, 6, 5
    r, k = torch.randn(n, dk, generator=g, dtype=torch.float64), torch.randn(n, dk, generator=g, dtype=torch.float64)
    v = torch.randn(n, dv, generator=g, dtype=torch.float64)
    decay = torch.rand(n, dk, generator=g, dtype=torch.float64) * 0.4 + 0.6
    rate = torch.rand(n, dk, generator=g, dtype=torch.float64)
    whole, S = plain.delta_rule_scan(r, k, v, decay, rate)
    a, Sa = plain.delta_rule_scan(r[:9], k[:9], v[:9], decay[:9], rate[:9])
    b, Sb = plain.delta_rule_scan(r[9:], k[9:], v[9:], decay[9:], rate[9:], state=Sa)
    assert torch.allclose(torch.cat([a, b]), whole, atol=1e-12) and torch.allclose(S, Sb, atol=1e-12)
    # a full removal rate with a unit decay replaces what the state held under this key
    k1 = torch.zeros(1, dk, dtype=torch.float64); k1[0, 2] = 3.0
    one = torch.ones(1, dk, dtype=torch.float64)
    _, S1 = plain.delta_rule_scan(k1, k1, torch.ones(1, dv, dtype=torch.float64), one, one)
    _, S2 = plain.delta_rule_scan(k1, k1, 2 * torch.ones(1, dv, dtype=torch.float64), one, one, state=S1)
    assert torch.allclose(S2[2], 6.0 * torch.ones(dv, dtype=torch.float64), atol=1e-5)
    h = torch.randn(7, 4, generator=g, dtype=torch.float64)
    mix = torch.rand(4, generator=g, dtype=torch.float64)
    whole = plain.token_shift(h, mix)
    cut = torch.cat([plain.token_shift(h[:3], mix), plain.token_shift(h[3:], mix, before=h[2])])
    assert torch.equal(whole, cut) and torch.allclose(whole[0], h[0] * (1 - mix), atol=1e-14)


def test_plain_chunk_edges():
    n, chunk = 25, 10
    q = torch.zeros(n, 1, 4, dtype=torch.float64)
    k = torch.zeros(n, 1, 4, dtype=torch.float64)
    v = torch.eye(n, dtype=torch.float64)[:, None, :]                  # value j is the j-th unit vector
    out = plain.chunked_sigmoid_attention(q, k, v, 1.0, torch.zeros(1, dtype=torch.float64), chunk)
    for i in range(n):
        seen = [j for j in range(n) if out[i, 0, j] != 0]
        assert seen == list(range(i // chunk * chunk, i + 1)) and all(out[i, 0, j] == 0.5 for j in seen)
