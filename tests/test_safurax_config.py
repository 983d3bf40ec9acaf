"""Host-side tests of the Safurax configuration, its model spec, tensor names and cache plan, and of the plain
implementation's mechanisms against library routines."""
import copy
import math

import pytest
import torch
import torch.nn.functional as F

import qwen_engine_amd  # noqa: F401
from qwen_engine_amd.cache import GroupSpec
from qwen_engine_amd.config import ConfigError, config_from_dict
from qwen_engine_amd.parts import cache_plan, expected_tensors
from qwen_engine_amd.weights.random_init import random_tensors
from plain import safurax_plain as S
from safurax_tiny import SA, SB, SC, TINY, tensor_shapes


@pytest.mark.parametrize("which", sorted(TINY))
def test_expected_tensors_are_the_designs_names(which):
    cfg = TINY[which][0]
    spec = config_from_dict(cfg).to_model_spec()
    want = {k: tuple(v[0]) for k, v in tensor_shapes(cfg).items()}
    got = {k: tuple(v.shape) for k, v in expected_tensors(spec).items() if not v.optional}
    assert got == want
    assert not spec.tie_head and spec.head_name == "head" and spec.final_norm_name == "final.norm"


def test_spec_and_cache_plan_follow_the_configuration():
    spec = config_from_dict(SA).to_model_spec()
    assert [l.prefix for l in spec.layers] == ["l0", "l1", "l2", "l3", "l4"]
    assert [(e.layer, e.cache_from) for e in spec.schedule] == [(0, None), (1, None), (2, None), (3, 1), (4, 1)]
    assert spec.stream_prologue.scale == 3.0
    m = [l.mixer for l in spec.layers]
    assert [x.kind for x in m] == ["latent_attention", "latent_attention", "diff_attention", "latent_attention", "latent_attention"]
    # the first kind: a query latent, no rotated part, every key, no sink, no gate
    assert (m[0].q_rank, m[0].rot_dim, m[0].window, m[0].sink, m[0].output_gate, m[0].position) == (56, 0, None, False, False, None)
    # the second: direct queries, a window, a sink, a gate per head, a half-split rotation of the whole rotated part
    assert (m[1].q_rank, m[1].rot_dim, m[1].window, m[1].sink, m[1].output_gate, m[1].gate_per_head) == (None, 12, 37, True, True, True)
    assert m[1].position.kind == "rope_half_angles" and m[1].position.rotary_dim == 12 and m[1].position.scaling_factor == 1.0
    # layer 1 keeps the widest window of itself and its readers; the readers keep nothing
    assert m[1].keep_window == 50 and (m[3].own_latent, m[4].own_latent) == (False, False)
    assert (m[3].window, m[4].window) == (50, 9)
    assert (m[2].num_heads, m[2].num_kv_heads, m[2].head_dim, m[2].v_head_dim, m[2].diff) == (4, 2, 16, 24, 0.3)
    assert m[2].position.scaling_factor == 4.0 and m[2].position.rotary_dim == 8 and m[2].qk_norm_eps == 1e-6
    assert spec.layers[3].ffn is None and spec.layers[3].ffn_norm is None
    f = spec.layers[1].ffn
    assert (f.kind, f.num_experts, f.top, f.intermediate_size, f.shared_intermediate_size, f.shared_gate, f.router_bias) == \
        ("top_softmax_moe", 6, 2, 40, 56, True, True)
    assert spec.layers[0].ffn.names == ("gate", "up", "down")
    plan = cache_plan(spec)
    assert plan.groups == [GroupSpec(None, 0), GroupSpec(50, 0)]
    assert plan.user_group == [0, 1, 0, 1, 1] and plan.user_source == [0, 1, 2, 1, 1]
    # one row of latent and rotated part a token; the two maps of differential attention as two key/value heads
    assert [(kv.num_kv_heads, kv.head_dim, kv.planes) if kv else None for kv in plan.user_kv] == \
        [(1, 40, 1), (1, 36, 1), (4, 64, 2), None, None]
    # no shared expert where the configuration names none; an embedding scale of one is no part at all
    spec_b = config_from_dict(SB).to_model_spec()
    assert spec_b.layers[0].ffn.shared_intermediate_size is None and spec_b.stream_prologue is None
    assert spec_b.layers[1].mixer.keep_window is None
    assert config_from_dict(SC).to_model_spec().layers[1].mixer.position is None


def test_config_errors_name_the_key():
    for path, message in ((("norm", "eps"), "norm.eps"), (("embedding", "scale"), "embedding.scale"),
                          (("layers", 2, "mixer", "kv_heads"), "layers[2].mixer.kv_heads"),
                          (("layers", 2, "mixer", "diff"), "layers[2].mixer.diff"),
                          (("layers", 1, "mixer", "mask", "size"), "layers[1].mixer.mask.size"),
                          (("layers", 0, "mixer", "q_rank"), "layers[0].mixer.q_rank"),
                          (("layers", 1, "mlp", "router", "top"), "router.top"),
                          (("layers", 1, "mlp", "shared", "ff"), "shared.ff")):
        d = copy.deepcopy(SA)
        cur = d
        for k in path[:-1]:
            cur = cur[k]
        del cur[path[-1]]
        with pytest.raises(ConfigError, match=message.replace("[", r"\[").replace("]", r"\]")):
            config_from_dict(d)
    for change, message in ((lambda d: d["layers"][3]["mixer"].update(kv_from=4), "kv_from"),
                            (lambda d: d["layers"][3]["mixer"].update(kv_from=0), "kv_from"),
                            (lambda d: d["layers"][4]["mixer"].update(kv_from=3), "kv_from"),
                            (lambda d: d["layers"][3]["mixer"].update(kv_rank=32), "kv_rank"),
                            (lambda d: d["layers"][3]["mixer"]["rot"].update(base=1.0), "rot"),
                            (lambda d: d["layers"][2]["mixer"].update(kv_heads=3), "multiple"),
                            (lambda d: d["layers"][2]["mixer"]["rot"].update(dims=18), "rot.dims"),
                            (lambda d: d["layers"][4]["mlp"]["router"].update(top=6), "top 6 of 5"),
                            (lambda d: d["layers"][0].update(type="mamba"), "type")):
        d = copy.deepcopy(SA)
        change(d)
        with pytest.raises(ConfigError, match=message):
            config_from_dict(d)


def test_random_weights_mode_writes_every_tensor():
    cfg = config_from_dict(SA)
    got = random_tensors(cfg, seed=5)
    assert {k: tuple(v.shape) for k, v in got.items()} == {k: tuple(v[0]) for k, v in tensor_shapes(SA).items()}


# ---- the plain implementation's mechanisms against library routines ----------------------------------------------
def test_plain_norms():
    g = torch.Generator().manual_seed(1)
    x = torch.randn(5, 48, generator=g, dtype=torch.float64) + 0.7
    w = torch.randn(48, generator=g, dtype=torch.float64)
    assert torch.allclose(S.layer_norm(x, w, 1e-5), F.layer_norm(x, (48,), w, None, 1e-5), atol=1e-12)
    assert torch.allclose(S.rms_norm(x, w, 1e-5), x / torch.sqrt((x * x).mean(-1, keepdim=True) + 1e-5) * w, atol=1e-12)


def test_plain_rotation_is_a_rotation_by_the_scaled_angle():
    g = torch.Generator().manual_seed(2)
    v = torch.randn(7, 3, 10, generator=g, dtype=torch.float64)
    pos = torch.tensor([0, 1, 2, 5, 40, 41, 1000])
    out = S.rotate_half_split(v, pos, 100.0, 6, factor=4.0)
    assert torch.equal(out[..., 6:], v[..., 6:]) and torch.allclose(out[0], v[0])
    for i in range(3):
        a = pos.double() * 100.0 ** (-2.0 * i / 6) / 4.0
        z = torch.complex(v[..., i], v[..., i + 3]) * torch.polar(torch.ones_like(a), a)[:, None]
        assert torch.allclose(out[..., i], z.real, atol=1e-12) and torch.allclose(out[..., i + 3], z.imag, atol=1e-12)
    # relative: the product of a rotated query and key depends on the distance alone
    q, k = torch.randn(1, 6, generator=g, dtype=torch.float64), torch.randn(1, 6, generator=g, dtype=torch.float64)
    dot = lambda pq, pk: float((S.rotate_half_split(q, torch.tensor([pq]), 50.0, 6) * S.rotate_half_split(k, torch.tensor([pk]), 50.0, 6)).sum())
    assert abs(dot(17, 11) - dot(106, 100)) < 1e-9


def test_plain_softmax_with_a_window_and_a_sink():
    g = torch.Generator().manual_seed(3)
    s = torch.randn(2, 9, 9, generator=g, dtype=torch.float64)
    sink = torch.tensor([0.4, -1.3], dtype=torch.float64)
    ok = S.visible(9, 4)
    assert ok[5].tolist() == [False, False, True, True, True, True, False, False, False] and ok[0].sum() == 1
    p = S.masked_softmax(s, ok, sink)
    for h in range(2):
        for i in range(9):
            cols = [j for j in range(9) if ok[i, j]]
            ref = torch.softmax(torch.cat([s[h, i, cols], sink[h:h + 1]]), dim=0)      # the sink as one more column
            assert torch.allclose(p[h, i, cols], ref[:-1], atol=1e-12) and float(p[h, i].sum()) < 1.0
    assert torch.allclose(S.masked_softmax(s, S.visible(9, None)).sum(-1), torch.ones(2, 9, dtype=torch.float64))


def test_plain_routing_weighs_the_chosen_logits_alone():
    z = torch.tensor([[0.1, 2.0, -1.0, 1.5, 0.3]], dtype=torch.float64)
    ids, w = S.route(z, 2)
    assert ids.tolist() == [[1, 3]]
    assert torch.allclose(w, torch.tensor([[1 / (1 + math.exp(-0.5)), 1 / (1 + math.exp(0.5))]], dtype=torch.float64))


def test_plain_differential_attention_of_equal_maps_and_the_lambda():
    """With both maps' projections equal and lambda = 0 + diff, a1 = a2 and the head's output is (1 - diff) a1 before
    its norm: the norm then leaves unit_rms(a1) * (1 - diff)."""
    g = torch.Generator().manual_seed(4)
    T, W, H, G, d, dv = 6, 20, 2, 1, 4, 6
    m = {"heads": H, "kv_heads": G, "dim": d, "vdim": dv, "diff": 0.25, "scale": 0.5}
    r = lambda *s: torch.randn(*s, generator=g, dtype=torch.float64)
    q1, k1 = r(H, 1, d, W), r(G, 1, d, W)
    w = {"q": q1.expand(H, 2, d, W).reshape(H * 2 * d, W), "k": k1.expand(G, 2, d, W).reshape(G * 2 * d, W), "v": r(G * dv, W),
         "q.norm": torch.ones(d, dtype=torch.float64), "k.norm": torch.ones(d, dtype=torch.float64),
         "lq1": r(d), "lk1": r(d), "g": torch.zeros(H, W, dtype=torch.float64), "o": torch.eye(H * dv, dtype=torch.float64)}
    w["lq2"], w["lk2"] = w["lq1"], w["lk1"]
    assert abs(S.differential_lambda(w, "", 0.25) - 0.25) < 1e-12
    h = r(T, W)
    out = S.differential_attention(h, torch.arange(T), w, "", m, 1e-6).view(T, H, dv)
    # one map by hand
    q = S.rms_norm((h @ q1.reshape(H * d, W).T).view(T, H, d), torch.ones(d, dtype=torch.float64), 1e-6)
    k = S.rms_norm((h @ k1.reshape(G * d, W).T).view(T, G, d), torch.ones(d, dtype=torch.float64), 1e-6)
    v = (h @ w["v"].T).view(T, G, dv)
    for hh in range(H):
        s = (q[:, hh] @ k[:, 0].T * 0.5).masked_fill(~S.visible(T, None), -math.inf)
        a1 = torch.softmax(s, dim=-1) @ v[:, 0]
        want = S.rms_unit(0.75 * a1, 1e-6) * 0.75 * 0.5            # (a gate of zero is a half)
        assert torch.allclose(out[:, hh], want, atol=1e-10)
