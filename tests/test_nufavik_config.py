"""Host-side tests of the Nufavik configuration, its model spec, tensor names and cache plan, of the cache manager's
kept first pages, and of the plain implementation's mechanisms against library routines."""
import copy

import pytest
import torch
import torch.nn.functional as F

import qwen_engine_amd  # noqa: F401
from qwen_engine_amd.cache import CacheManager, GroupSpec, StateNeed
from qwen_engine_amd.config import ConfigError, config_from_dict
from qwen_engine_amd.parts import cache_plan, expected_tensors
from qwen_engine_amd.weights.random_init import random_tensors
from plain import nufavik_plain as N
from nufavik_tiny import NA, TINY, tensor_shapes


@pytest.mark.parametrize("which", sorted(TINY))
def test_expected_tensors_are_the_designs_names(which):
    cfg = TINY[which][0]
    spec = config_from_dict(cfg).to_model_spec()
    want = {k: tuple(v[0]) for k, v in tensor_shapes(cfg).items()}
    got = {k: tuple(v.shape) for k, v in expected_tensors(spec).items() if not v.optional}
    assert got == want
    assert spec.tie_head and spec.head_name == "embed"


def test_spec_and_cache_plan_follow_the_configuration():
    spec = config_from_dict(NA).to_model_spec()
    assert [l.prefix for l in spec.layers] == ["l0", "l1", "l2", "l3"] and [e.layer for e in spec.schedule] == [0, 1, 2, 3]
    assert spec.stream_prologue.scale == 0.7
    m = [l.mixer for l in spec.layers]
    assert [(a.window, a.keep_first, a.conv_taps, a.sink) for a in m] == [(24, 3, 3, True), (7, 0, 2, True), (37, 20, 5, True), (9, 12, 4, True)]
    assert m[2].position is None and m[1].position.rotary_dim == 24 and m[0].position.theta == 1000.0
    assert spec.layers[1].ffn is None and spec.layers[2].ffn.num_identity == 1 and spec.layers[3].ffn.route_scale == 2.0
    plan = cache_plan(spec)
    assert plan.groups == [GroupSpec(24, 3), GroupSpec(7, 0), GroupSpec(37, 20), GroupSpec(9, 12)]
    # keys and values of different sizes share the cache under one head size
    assert [(kv.num_kv_heads, kv.head_dim) for kv in plan.user_kv] == [(2, 64), (3, 64), (1, 64), (1, 64)]
    # the state: the last taps - 1 projected rows of q | k | v
    assert plan.user_state == [StateNeed(shape=(2, 4 * 16 + 2 * 16 + 2 * 24)), StateNeed(shape=(1, 3 * 24 + 3 * 24 + 3 * 8)),
                               StateNeed(shape=(4, 6 * 8 + 8 + 40)), StateNeed(shape=(3, 2 * 32 + 32 + 16))]
    d = copy.deepcopy(NA)
    d["embedding"]["scale"] = 1.0
    assert config_from_dict(d).to_model_spec().stream_prologue is None


def test_config_errors_name_the_key():
    for path, message in ((("norm", "eps"), "norm.eps"), (("embedding", "scale"), "embedding.scale"),
                          (("layers", 1, "mixer", "kv_heads"), "layers[1].mixer.kv_heads"),
                          (("layers", 0, "mixer", "mask", "keep_first"), "layers[0].mixer.mask.keep_first"),
                          (("layers", 2, "mlp", "router", "identity"), "router.identity")):
        d = copy.deepcopy(NA)
        cur = d
        for k in path[:-1]:
            cur = cur[k]
        del cur[path[-1]]
        with pytest.raises(ConfigError, match=message.replace("[", r"\[").replace("]", r"\]")):
            config_from_dict(d)
    d = copy.deepcopy(NA)
    d["layers"][2]["mlp"]["router"]["top"] = 5          # three experts and one identity expert hold four
    with pytest.raises(ConfigError, match="cannot be chosen"):
        config_from_dict(d)
    d = copy.deepcopy(NA)
    d["layers"][0]["type"] = "latent_attention"
    with pytest.raises(ConfigError, match="type"):
        config_from_dict(d)
    d = copy.deepcopy(NA)
    d["layers"][0]["mixer"]["rot"]["dims"] = 18
    with pytest.raises(ConfigError, match="rot.dims"):
        config_from_dict(d)


def test_random_weights_mode_writes_every_tensor():
    cfg = config_from_dict(NA)
    got = random_tensors(cfg, seed=5)
    assert {k: tuple(v.shape) for k, v in got.items()} == {k: tuple(v[0]) for k, v in tensor_shapes(NA).items()}


# ---- the cache manager: a window that keeps the first keys' pages ----------------------------------------------
def test_pages_of_the_kept_first_keys_stay_while_the_window_moves_on():
    P = 4
    cm = CacheManager([GroupSpec(window=6, keep_first=5), GroupSpec(window=6), GroupSpec()], [12, 12, 12], P, 2)
    cm.add_request("a")
    for n in (3, 7, 2, 1, 1, 9, 1):
        rc = cm.get("a")
        cm.reserve("a", rc.num_tokens + n)
        cm.commit("a", [0] * n)
        cm.check_invariants()
        first_live = max(0, cm.get("a").num_tokens - 6 + 1) // P
        for g, kept in ((0, 2), (1, 0)):
            held = [i for i, pg in enumerate(cm.block_table("a", g)) if pg >= 0]
            n_table = len(cm.block_table("a", g))
            want = sorted(set(range(min(kept, n_table))) | set(range(first_live, n_table)))
            assert held == want, (g, cm.get("a").num_tokens, held, want)
        assert all(pg >= 0 for pg in cm.block_table("a", 2))
    free_before = [p.num_free for p in cm.pools]
    cm.free_request("a")
    cm.check_invariants()
    assert [p.num_free for p in cm.pools] == [12, 12, 12] and free_before[0] < free_before[1]


# ---- the plain implementation's mechanisms against library routines ------------------------------------------------
def test_plain_convolution_is_a_causal_depthwise_convolution():
    g = torch.Generator().manual_seed(1)
    u, w = torch.randn(19, 7, generator=g, dtype=torch.float64), torch.randn(7, 4, generator=g, dtype=torch.float64)
    want = F.conv1d(F.pad(u.T.unsqueeze(0), (3, 0)), w.unsqueeze(1), groups=7)[0].T
    assert torch.allclose(N.causal_conv(u, w), want, atol=1e-12)


def test_plain_rotation_is_a_complex_product_on_split_halves():
    g = torch.Generator().manual_seed(2)
    v = torch.randn(9, 3, 16, generator=g, dtype=torch.float64)
    pos = torch.arange(4, 13)
    got = N.rotate_half_split(v, pos, 100.0, 12)
    z = torch.complex(v[..., :6], v[..., 6:12])
    ang = pos.double().reshape(-1, 1, 1) * (100.0 ** (-torch.arange(6, dtype=torch.float64) / 6))
    want = z * torch.polar(torch.ones_like(ang), ang)
    assert torch.allclose(got[..., :6], want.real, atol=1e-12) and torch.allclose(got[..., 6:12], want.imag, atol=1e-12)
    assert torch.equal(got[..., 12:], v[..., 12:])


def test_plain_softmax_with_a_sink_is_a_softmax_over_one_more_zero():
    s = torch.tensor([0.3, -2.0, 4.1, 0.0], dtype=torch.float64)
    want = torch.softmax(torch.cat([s, torch.zeros(1, dtype=torch.float64)]), 0)[:4]
    assert torch.allclose(N.softmax_with_sink(s), want, atol=1e-14)
    assert float(N.softmax_with_sink(torch.tensor([-50.0], dtype=torch.float64))) < 1e-20


def test_plain_mask_is_a_window_and_the_first_keys():
    seen = [[j for j in range(12) if N.sees(i, j, 3, 2)] for i in range(12)]
    assert seen[0] == [0] and seen[2] == [0, 1, 2] and seen[4] == [0, 1, 2, 3, 4] and seen[5] == [0, 1, 3, 4, 5]
    assert seen[11] == [0, 1, 9, 10, 11]


def test_plain_router_chooses_by_corrected_scores_and_weighs_by_the_scores():
    z = torch.tensor([1.0, 2.0, 0.5, 1.9], dtype=torch.float64)
    s = torch.softmax(z, 0)
    ids, w = N.route(z, torch.zeros(4, dtype=torch.float64), 2, 3.0)
    assert ids == [1, 3] and torch.allclose(w, 3.0 * s[[1, 3]] / (s[1] + s[3]))
    ids, w = N.route(z, torch.tensor([0.0, -1.0, 1.0, 0.0], dtype=torch.float64), 2, 3.0)
    assert ids == [2, 3] and torch.allclose(w, 3.0 * s[[2, 3]] / (s[2] + s[3]))     # the correction chooses, the scores weigh
    ids, _ = N.route(torch.zeros(4, dtype=torch.float64), torch.zeros(4, dtype=torch.float64), 3, 1.0)
    assert ids == [0, 1, 2]                                                         # the lower index on ties
