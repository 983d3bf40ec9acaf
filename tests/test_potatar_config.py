"""Host-side tests of the Potatar configuration, its model spec, tensor names and cache plan, and of the plain
implementation's mechanisms against library routines."""
import copy
import json
import math

import pytest
import torch
import torch.nn.functional as F

import qwen_engine_amd  # noqa: F401
from qwen_engine_amd.config import ConfigError, config_from_dict
from qwen_engine_amd.parts import cache_plan, expected_tensors
from plain import potatar_plain as N
from potatar_tiny import PA, PB, PC, SHAPE_SIZES, TINY, make_folder, random_tensors, tensor_shapes


def _shapes(which):
    return {k: tuple(v[0]) for k, v in tensor_shapes(TINY[which][0]).items()}


@pytest.mark.parametrize("which", sorted(TINY))
def test_expected_tensors_are_the_designs_names(which):
    cfg = TINY[which][0]
    want = _shapes(which)
    spec = config_from_dict(cfg, shapes=want).to_model_spec()
    got = {k: tuple(v.shape) for k, v in expected_tensors(spec).items() if not v.optional}
    assert got == want
    assert not spec.tie_head and spec.head_name == "head"


def test_spec_and_cache_plan_follow_the_configuration():
    spec = config_from_dict(PA, shapes=_shapes("A")).to_model_spec()
    assert [l.prefix for l in spec.layers] == [f"l{i}" for i in range(6)] and [e.layer for e in spec.schedule] == list(range(6))
    assert all(l.alpha == 1.7 for l in spec.layers) and spec.logit_epilogue.cap == 9.0
    m = [l.mixer for l in spec.layers]
    assert (m[0].num_heads, m[0].head_dim, m[0].decay_rank) == (3, 8, 5)
    att = [m[1], m[3], m[4], m[5]]
    assert [a.chunk for a in att] == [13, 7, 64, 9]
    assert [a.value_blend for a in att] == ["source", "blend", None, "blend"]       # the first blending layer only gives
    assert att[2].position is None and att[0].position.rotary_dim == 4 and att[1].position.theta == 50000.0
    assert all(a.qk_norm == "whole" and a.bias for a in att)
    left, right = m[2].left, m[2].right
    assert (left.qk_norm, left.values_from_keys, left.talking_heads, left.distance_bias_rows, left.distance_bias_far, left.chunk) == \
        ("head", True, True, 10, 30.0, 21)
    assert right.decay == (0.5, 0.93) and (right.num_heads, right.head_dim, right.v_head_dim) == (2, 12, 8)
    assert (m[2].left_scale, m[2].right_scale) == (0.7, 1.3)
    assert [l.ffn is None for l in spec.layers] == [False, False, True, False, True, False]
    plan = cache_plan(spec)
    # the attention layers keep every key (a chunk's first keys are read until it ends); the others have a state
    assert [kv.num_kv_heads for kv in plan.user_kv if kv is not None] == [2, 3, 2, 3, 2]
    states = [s for s in plan.user_state if s is not None]
    assert [s.shape for s in states] == [(80 + 3 * 8 * 8,), (2 * 12 * 8,)] and all(s.dtype == "float32" for s in states)


def test_sizes_that_only_tensor_shapes_give():
    cfg = config_from_dict(PA, shapes=_shapes("A"))
    d = cfg.to_dict()
    assert d["layers"][0]["mixer"]["decay_rank"] == 5 and d["layers"][2]["mixer"]["left"]["bias_rows"] == 10
    config_from_dict(d).to_model_spec()                                   # (a dictionary that names them needs no shapes)
    with pytest.raises(ConfigError, match="decay_rank"):
        config_from_dict(PA)
    assert "decay_rank" not in PA["layers"][0]["mixer"]                   # (the caller's dictionary is left as it was)


def test_the_loader_reads_them_from_the_file(tmp_path):
    from qwen_engine_amd.config import config_from_folder as load_config
    folder = make_folder(tmp_path, "C")
    cfg = load_config(folder)
    assert cfg.architecture == "Potatar"
    d = cfg.to_dict()
    assert d["layers"][1]["mixer"]["left"]["bias_rows"] == 2 and d["layers"][2]["mixer"]["decay_rank"] == 1
    assert d["layers"][4]["mixer"]["left"]["bias_rows"] == 33


def test_config_errors_name_the_key():
    shapes = _shapes("A")
    for path, message in ((("norm", "eps"), "norm.eps"), (("postln_alpha",), "postln_alpha"), (("width",), "width"),
                          (("layers", 1, "mixer", "kv_heads"), "layers[1].mixer.kv_heads"),
                          (("layers", 1, "mixer", "scale"), "layers[1].mixer.scale"),
                          (("layers", 2, "mixer", "left", "bias_max"), "layers[2].mixer.left.bias_max"),
                          (("layers", 2, "mixer", "right", "decay"), "layers[2].mixer.right.decay"),
                          (("layers", 2, "mixer", "right_scale"), "layers[2].mixer.right_scale"),
                          (("layers", 1, "mlp", "ff"), "layers[1].mlp.ff")):
        d = copy.deepcopy(PA)
        cur = d
        for k in path[:-1]:
            cur = cur[k]
        del cur[path[-1]]
        with pytest.raises(ConfigError, match=message.replace("[", r"\[").replace("]", r"\]")):
            config_from_dict(d, shapes=shapes)
    for path, value in ((("layers", 1, "mixer", "kv_heads"), 3), (("layers", 1, "mixer", "rot", "dims"), 5),
                        (("layers", 1, "mixer", "rot", "dims"), 14), (("layers", 2, "mixer", "right", "decay"), [0.5]),
                        (("layers", 3, "mixer", "mask", "size"), 0), (("layers", 0, "type"), "conv"),
                        (("layers", 1, "mlp", "kind"), "moe"), (("layers", 2, "mixer", "left", "vdim"), 9),
                        (("layers", 3, "mixer", "vdim"), 10)):            # (values of another size than the first blending layer's)
        d = copy.deepcopy(PA)
        cur = d
        for k in path[:-1]:
            cur = cur[k]
        cur[path[-1]] = value
        with pytest.raises(ConfigError):
            config_from_dict(d, shapes=shapes)


def test_random_weights_for_a_configuration_have_every_tensor():
    from qwen_engine_amd.weights.random_init import random_tensors as engine_random
    t = engine_random(config_from_dict(PB, shapes=_shapes("B")), seed=1)
    assert {k: tuple(v.shape) for k, v in t.items()} == _shapes("B")


# ---- the plain implementation's mechanisms against library routines ------------------------------------------------
def test_plain_norm_activations_and_softmax():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(5, 32, generator=g, dtype=torch.float64)
    w = torch.randn(32, generator=g, dtype=torch.float64)
    assert torch.allclose(N.rms_norm(x, w, 1e-5), F.rms_norm(x, (32,), w, 1e-5))
    assert torch.allclose(N.gelu_erf(x), F.gelu(x))
    assert torch.allclose(N.silu(x), F.silu(x)) and torch.allclose(N.sigmoid(x), torch.sigmoid(x))
    assert torch.allclose(N.softmax_rows(x), torch.softmax(x, -1))


def test_plain_rotation_turns_pairs_by_the_position():
    v = torch.zeros(3, 1, 8, dtype=torch.float64)
    v[:, 0, 1] = 1.0                      # coordinate 1 is paired with 1 + dims / 2 = 4
    v[:, 0, 7] = 2.0                      # beyond dims: stays
    out = N.rotate_half_split(v, torch.tensor([0, 1, 5]), 100.0, 6)
    for row, p in zip(out, (0, 1, 5)):
        a = p * 100.0 ** (-2.0 / 6)
        assert torch.allclose(row[0], torch.tensor([0, math.cos(a), 0, 0, math.sin(a), 0, 0, 2.0], dtype=torch.float64))


def test_plain_chunks_and_distance_rows():
    assert [j for j in range(12) if N.sees(9, j, 4)] == [8, 9] and [j for j in range(12) if N.sees(7, j, 4)] == [4, 5, 6, 7]
    assert [j for j in range(5) if N.sees(3, j, 1)] == [3]
    rows = [N.distance_bucket(n, 8, 64) for n in range(70)]
    assert rows[:4] == [0, 1, 2, 3] and rows[4] == 4 and rows[7] == 4 and rows[8] == 5 and rows[15] == 5 and rows[16] == 6
    assert rows[31] == 6 and rows[32] == 7 and rows[63] == 7 and rows[64] == 7 and rows[69] == 7
    assert rows == sorted(rows)


def test_plain_chunk_attention_is_softmax_attention_inside_each_chunk():
    g = torch.Generator().manual_seed(1)
    T, H, G, D = 11, 4, 2, 6
    q, k, v = (torch.randn(T, h, D, generator=g, dtype=torch.float64) for h in (H, G, G))
    got = N.chunk_attention(q, k, v, torch.arange(T), 0.4, 4)
    for lo in range(0, T, 4):
        hi = min(lo + 4, T)
        kk, vv = (t[lo:hi].repeat_interleave(H // G, dim=1).transpose(0, 1) for t in (k, v))
        want = F.scaled_dot_product_attention(q[lo:hi].transpose(0, 1), kk, vv, is_causal=True, scale=0.4).transpose(0, 1)
        assert torch.allclose(got[lo:hi], want)
    # an identity that mixes nothing and a bias of zeros change nothing; a bias on distance 0 alone sharpens the diagonal
    same = N.chunk_attention(q, k, v, torch.arange(T), 0.4, 4, bias=torch.zeros(6, H, dtype=torch.float64), far=10.0,
                             talk=torch.eye(H, dtype=torch.float64))
    assert torch.allclose(same, got)
    bias = torch.zeros(6, H, dtype=torch.float64)
    bias[0] = 50.0
    own = N.chunk_attention(q, k, v, torch.arange(T), 0.4, 4, bias=bias, far=10.0)
    assert torch.allclose(own, v.repeat_interleave(H // G, dim=1), atol=1e-9)
    # heads swapped by the mixing matrix swap their weights (the values stay each head's own)
    swap = torch.eye(H, dtype=torch.float64)[[1, 0, 3, 2]]
    sw = N.chunk_attention(q, k, v, torch.arange(T), 0.4, 4, talk=swap)
    assert torch.allclose(sw, N.chunk_attention(q[:, [1, 0, 3, 2]], k, v, torch.arange(T), 0.4, 4))


def test_plain_recurrences_are_their_sums():
    g = torch.Generator().manual_seed(2)
    T, H, D, Dv = 7, 2, 3, 4
    q, k = (torch.randn(T, H, D, generator=g, dtype=torch.float64) for _ in range(2))
    v = torch.randn(T, H, Dv, generator=g, dtype=torch.float64)
    dec = torch.tensor([0.5, 1.0], dtype=torch.float64)
    got = N.decayed_sum_state(q, k, v, dec)
    for t in range(T):
        for h in range(H):
            want = sum(float(dec[h]) ** (t - s) * float(q[t, h] @ k[s, h]) * v[s, h] for s in range(t + 1))
            assert torch.allclose(got[t, h], want)
    w = torch.rand(T, H, D, generator=g, dtype=torch.float64)
    u = torch.randn(H, D, generator=g, dtype=torch.float64)
    vv = torch.randn(T, H, D, generator=g, dtype=torch.float64)
    got = N.bonus_state(q, k, vv, w, u)
    for t in range(T):
        for h in range(H):
            want = float((q[t, h] * u[h]) @ k[t, h]) * vv[t, h]
            for s in range(t):
                between = torch.ones(D, dtype=torch.float64)
                for r in range(s + 1, t):
                    between = between * w[r, h]
                want = want + float((q[t, h] * between) @ k[s, h]) * vv[s, h]
            assert torch.allclose(got[t, h], want)


def test_plain_model_runs_every_tiny_configuration(tmp_path):
    for which in TINY:
        cfg, w = N.read_folder(make_folder(tmp_path, which))
        layers = []
        logits = N.forward(cfg, w, [1, 5, 9, 2, 7], layers_out=layers)
        assert logits.shape == (5, cfg["vocab"]) and len(layers) == len(cfg["layers"])
        assert float(logits.abs().max()) <= cfg["logit_softcap"] and not torch.isnan(logits).any()
        # a later token changes nothing before it
        again = N.forward(cfg, w, [1, 5, 9, 3, 7])
        assert torch.equal(again[:3], logits[:3]) and not torch.equal(again[3], logits[3])
