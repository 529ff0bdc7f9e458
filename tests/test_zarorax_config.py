"""Host-side tests of the Zarorax configuration, its model spec, tensor names and cache plan, and of the
plain implementation's mechanisms against library routines."""
import copy
import math

import pytest
import torch
import torch.nn.functional as F

import qwen_engine_amd  # noqa: F401
from qwen_engine_amd.cache import StateNeed
from qwen_engine_amd.config import ConfigError, config_from_dict
from qwen_engine_amd.parts import cache_plan, expected_tensors
from qwen_engine_amd.weights.random_init import random_tensors
from plain import zarorax_plain as Z
from zarorax_tiny import TINY, ZP, tensor_shapes


@pytest.mark.parametrize("which", sorted(TINY))
def test_expected_tensors_are_the_designs_names(which):
    cfg = TINY[which][0]
    spec = config_from_dict(cfg).to_model_spec()
    want = {k: tuple(v[0]) for k, v in tensor_shapes(cfg).items()}
    got = {k: tuple(v.shape) for k, v in expected_tensors(spec).items() if not v.optional}
    assert got == want


def test_schedule_runs_shared_layers_again_with_caches_of_their_own():
    spec = config_from_dict(ZP).to_model_spec()
    assert [e.layer for e in spec.schedule] == [0, 1, 0, 2]
    assert [l.prefix for l in spec.layers] == ["l0", "l1", "l3"]
    plan = cache_plan(spec)
    assert plan.entry_users == [[0], [1], [2], [3]] and plan.user_source == [0, 1, 2, 3]
    assert [(kv.num_kv_heads, kv.head_dim, kv.planes) for kv in plan.user_kv] == [(1, 48, 1), (1, 36, 1), (1, 48, 1), (1, 76, 1)]
    assert plan.user_state == [StateNeed(shape=(2, 96))] * 4
    assert plan.bytes_per_token(2) == 2 * (48 + 36 + 48 + 76)
    assert spec.layers[2].ffn is None and spec.layers[0].mixer.q_rank == 56 and spec.layers[1].mixer.output_gate


def test_config_errors_name_the_key():
    for path, message in ((("norm", "eps"), "norm.eps"), (("layers", 1, "mixer", "kv_rank"), "layers[1].mixer.kv_rank"),
                          (("layers", 0, "mixer", "q_rank"), "layers[0].mixer.q_rank"),
                          (("layers", 1, "mlp", "router", "top"), "router.top")):
        d = copy.deepcopy(ZP)
        cur = d
        for k in path[:-1]:
            cur = cur[k]
        del cur[path[-1]]
        with pytest.raises(ConfigError, match=message.replace("[", r"\[").replace("]", r"\]")):
            config_from_dict(d)
    d = copy.deepcopy(ZP)
    d["layers"][2]["weights_of"] = 2
    with pytest.raises(ConfigError, match="weights_of"):
        config_from_dict(d)
    d = copy.deepcopy(ZP)
    d["layers"][1]["mlp"]["router"]["top"] = 5          # two groups of two experts hold four
    with pytest.raises(ConfigError, match="cannot be chosen"):
        config_from_dict(d)
    d = copy.deepcopy(ZP)
    d["layers"][0]["type"] = "attention"
    with pytest.raises(ConfigError, match="type"):
        config_from_dict(d)


def test_random_weights_mode_writes_every_tensor():
    cfg = config_from_dict(ZP)
    t = random_tensors(cfg, seed=3)
    assert set(t) == set(tensor_shapes(ZP))
    assert t["final.norm"].shape == () and float(t["l0.norm1"]) == 1.0


# ---- the plain implementation's mechanisms against library routines -------------------------------------
def test_plain_convolution_is_a_causal_depthwise_convolution_plus_its_input():
    g = torch.Generator().manual_seed(0)
    h, w = torch.randn(9, 5, generator=g, dtype=torch.float64), torch.randn(5, 4, generator=g, dtype=torch.float64)
    want = h + F.conv1d(F.pad(h.t()[None], (3, 0)), w[:, None, :], groups=5)[0].t()
    assert torch.allclose(Z.short_conv(h, w), want, atol=1e-12)


def test_plain_rotation_is_a_complex_product_on_neighbouring_pairs():
    g = torch.Generator().manual_seed(1)
    v = torch.randn(7, 3, 10, generator=g, dtype=torch.float64)
    pos = torch.tensor([0, 1, 2, 50, 51, 700, 701])
    out = Z.rotate_interleaved(v, pos, 1000.0, 6)
    z = torch.view_as_complex(v[..., :6].reshape(7, 3, 3, 2).contiguous())
    ang = pos[:, None].double() * (1000.0 ** (-torch.arange(3).double() * 2 / 6))[None]
    want = torch.view_as_real(z * torch.polar(torch.ones_like(ang), ang)[:, None]).reshape(7, 3, 6)
    assert torch.allclose(out[..., :6], want, atol=1e-12) and torch.equal(out[..., 6:], v[..., 6:])


def test_plain_router_keeps_the_best_groups_and_unnormalised_scores():
    r = {"experts": 6, "top": 2, "groups": {"count": 3, "keep": 2}}
    router = torch.eye(6, dtype=torch.float64)
    # scores rise with the logits: group 0 = (0.1, 3.0), group 1 = (2.0, 2.5), group 2 = (2.9, 0.2)
    h = torch.tensor([[0.1, 3.0, 2.0, 2.5, 2.9, 0.2]], dtype=torch.float64)
    (picks,) = Z.route(h, router, r)
    s = torch.softmax(h[0], 0)
    assert [e for e, _ in picks] == [1, 4]               # not 3: its group is the third best
    assert picks[0][1] == pytest.approx(float(s[1])) and picks[1][1] == pytest.approx(float(s[4]))
    assert sum(w for _, w in picks) < 1.0


def test_plain_attention_of_one_head_is_library_attention_over_expanded_keys():
    cfg, seed, _ = TINY["P"]
    from zarorax_tiny import random_tensors as rt
    w = {k: v.double() for k, v in rt(cfg, seed).items()}
    m = cfg["layers"][3]["mixer"]
    g = torch.Generator().manual_seed(2)
    h = torch.randn(6, cfg["width"], generator=g, dtype=torch.float64)
    pos = torch.arange(6)
    got = Z.latent_attention(h, pos, w, "l3.mix", m, 1e-6, gated=True)
    H, dn, dr, dv, r = m["heads"], m["dim"], m["rot_dim"], m["vdim"], m["kv_rank"]
    q = (h @ w["l3.mix.q"].t()).view(6, H, dn + dr)
    kv = h @ w["l3.mix.dkv"].t()
    c = F.rms_norm(kv[:, :r], (r,), weight=w["l3.mix.dkv.norm"], eps=1e-6)
    kr = Z.rotate_interleaved(kv[:, r:], pos, m["rot"]["base"], m["rot"]["dims"])
    qr = Z.rotate_interleaved(q[..., dn:], pos, m["rot"]["base"], m["rot"]["dims"])
    k = torch.cat([(c @ w["l3.mix.uk"].t()).view(6, H, dn), kr[:, None].expand(6, H, dr)], -1)
    v = (c @ w["l3.mix.uv"].t()).view(6, H, dv)
    o = F.scaled_dot_product_attention(torch.cat([q[..., :dn], qr], -1).transpose(0, 1)[None], k.transpose(0, 1)[None],
                                       v.transpose(0, 1)[None], is_causal=True, scale=m["scale"])[0].transpose(0, 1)
    want = (o.reshape(6, H * dv) * torch.sigmoid(h @ w["l3.mix.g"].t())) @ w["l3.mix.o"].t()
    assert torch.allclose(got, want, atol=1e-10)
