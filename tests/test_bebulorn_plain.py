"""The plain implementation of the Bebulorn design against forms written another way (sums over all earlier tokens,
loops, hand-made cases), and the typed configuration: run order, tensor names, what the cache manager is asked for,
refusals.  No GPU."""
import copy
import math

import numpy as np
import pytest

from tests.plain import bebulorn_plain as P

RNG = np.random.default_rng(7)


def test_layer_norm_by_hand():
    x = np.array([[1.0, 2.0, 3.0, 6.0]])
    w, b = np.array([1.0, 2.0, 0.5, 1.0]), np.array([0.0, 1.0, 0.0, -1.0])
    mean, var = 3.0, (4 + 1 + 0 + 9) / 4
    ref = (x - mean) / math.sqrt(var + 0.1) * w + b
    assert np.allclose(P.layer_norm(x, w, b, 0.1), ref)
    assert np.allclose(P.rms(np.array([3.0, 4.0]), 0.5), np.array([3.0, 4.0]) / math.sqrt(12.5 + 0.5))


def test_decay_scan_is_the_weighted_sum_over_all_earlier_tokens_and_carries_its_state():
    T, H, d, dv = 9, 2, 3, 4
    q, k, v = RNG.normal(size=(T, H, d)), RNG.normal(size=(T, H, d)), RNG.normal(size=(T, H, dv))
    decay = np.array([0.5, 1.0])
    o, s = P.lightning_scan(q, k, v, decay)
    for t in range(T):
        for h in range(H):
            ref = sum(decay[h] ** (t - j) * (q[t, h] @ k[j, h]) * v[j, h] for j in range(t + 1))
            assert np.allclose(o[t, h], ref)
    o1, s1 = P.lightning_scan(q[:4], k[:4], v[:4], decay)
    o2, s2 = P.lightning_scan(q[4:], k[4:], v[4:], decay, state=s1)
    assert np.allclose(np.concatenate([o1, o2]), o) and np.allclose(s2, s)


def test_delta_rule_writes_before_it_reads_and_forgets_by_its_gate():
    d, dv = 4, 3
    k = np.zeros((2, 1, d)); k[0, 0, 0] = 1.0; k[1, 0, 0] = 1.0
    v = RNG.normal(size=(2, 1, dv))
    q = k.copy()
    # beta 1 and no forgetting: the read-out at a token's own key is its own value, also when the key was written before
    o, s = P.delta_scan(q, k, v, np.ones((2, 1)), np.ones((2, 1)))
    assert np.allclose(o[0, 0], v[0, 0]) and np.allclose(o[1, 0], v[1, 0])
    # beta 0 writes nothing; the gate alone shrinks what is there
    o, s = P.delta_scan(q, k, v, np.array([[1.0], [0.0]]), np.array([[1.0], [0.25]]))
    assert np.allclose(o[1, 0], 0.25 * v[0, 0])
    # across a cut with carried state
    T, H = 8, 2
    q, k, v = RNG.normal(size=(T, H, d)), RNG.normal(size=(T, H, d)), RNG.normal(size=(T, H, dv))
    beta, g = RNG.uniform(size=(T, H)), RNG.uniform(size=(T, H))
    o, s = P.delta_scan(q, k, v, beta, g)
    o1, s1 = P.delta_scan(q[:3], k[:3], v[:3], beta[:3], g[:3])
    o2, s2 = P.delta_scan(q[3:], k[3:], v[3:], beta[3:], g[3:], state=s1)
    assert np.allclose(np.concatenate([o1, o2]), o) and np.allclose(s2, s)


def test_short_convolution_by_hand_and_across_a_cut():
    x = np.arange(1.0, 7.0).reshape(6, 1)
    w = np.array([[100.0, 10.0, 1.0]])           # the last column is the current token's
    assert np.allclose(P.short_conv(x, w)[:, 0], [1, 12, 123, 234, 345, 456])
    x, w = RNG.normal(size=(10, 5)), RNG.normal(size=(5, 4))
    whole = P.short_conv(x, w)
    assert np.allclose(P.short_conv(x[6:], w, before=x[3:6]), whole[6:])
    assert np.allclose(P.short_conv(x[:6], w), whole[:6])
    assert np.allclose(P.short_conv(x, np.ones((5, 1))), x)      # one tap: the token itself


def test_window_mask_and_capped_scores():
    m = P.window_mask(6, 3)
    assert m[5].tolist() == [False, False, False, True, True, True] and m[1].tolist() == [True, True, False, False, False, False]
    assert P.window_mask(4, 1)[3].tolist() == [False, False, False, True] and P.window_mask(3, None)[2].all()
    # a changed token just outside the window changes nothing, just inside it does
    T, H, G, d = 12, 2, 1, 4
    q, k, v = RNG.normal(size=(T, H, d)), RNG.normal(size=(T, G, d)), RNG.normal(size=(T, G, d))
    base = P.capped_attention(q, k, v, G, 0.5, np.array([1.0, 2.0]), 5.0, 4)
    for j, changes in ((T - 5, False), (T - 4, True)):
        k2, v2 = k.copy(), v.copy()
        k2[j] += 3.0; v2[j] -= 2.0
        other = P.capped_attention(q, k2, v2, G, 0.5, np.array([1.0, 2.0]), 5.0, 4)
        assert (not np.allclose(other[T - 1], base[T - 1])) == changes
    # the cap bounds what a huge score can do: two keys with scores far above the cap weigh alike
    q1, k1 = np.full((2, 1, 1), 100.0), np.array([[[100.0]], [[200.0]]])
    out = P.capped_attention(q1, k1, np.array([[[0.0]], [[1.0]]]), 1, 1.0, np.array([1.0]), 2.0, None)
    assert abs(out[1, 0, 0] - 0.5) < 1e-6
    # the head's factor multiplies the score inside the cap
    one = P.capped_attention(q[:, :1], k, v, 1, 0.5, np.array([3.0]), 5.0, None)
    folded = P.capped_attention(q[:, :1] * 3.0, k, v, 1, 0.5, np.array([1.0]), 5.0, None)
    assert np.allclose(one, folded)


def test_route_picks_the_largest_and_weighs_them_over_their_sum():
    h = np.eye(4)
    w_router = np.array([[0.0, 3.0, 1.0, 0.0], [2.0, 0.0, 1.0, 0.0], [1.0, 1.0, 1.0, 0.0]])   # [experts, width]
    chosen, weights = P.route(h, w_router, 2)
    assert chosen[0].tolist() == [1, 2] and chosen[1].tolist() == [0, 2]
    assert chosen[2].tolist() == [0, 1] and chosen[3].tolist() == [0, 1]         # equal scores: the lower index first
    assert np.allclose(weights.sum(axis=1), 1.0)
    z = np.array([0.0, 2.0, 1.0])
    s = np.exp(z) / np.exp(z).sum()
    assert np.allclose(weights[0], [s[1] / (s[1] + s[2]), s[2] / (s[1] + s[2])])
    assert np.allclose(P.route(h, w_router, 3)[1][0], s[[1, 2, 0]])


def test_gelu_and_unit():
    assert abs(P.gelu_erf(1.0) - 0.8413447460685429) < 1e-12 and P.gelu_erf(0.0) == 0.0
    x = RNG.normal(size=(3, 5))
    assert np.allclose(np.sum(P.unit(x) ** 2, axis=-1), np.sum(x * x, axis=-1) / (np.sum(x * x, axis=-1) + 1e-6))


# ------------------------------------------------------------------------------------------------ configuration

def _config():
    from kipp_amd.config import shape_config
    return shape_config("bebulorn-tiny-a")


def test_run_order_and_tensor_names():
    from kipp_amd.config import parse_config
    from kipp_amd.engine.model import model_params
    d = _config()
    _, cfg = parse_config(d)
    spec = cfg.model_spec()
    assert [(r.layer, r.add_embedding) for r in spec.order] == [(0, False), (1, False), (0, True), (1, False), (0, True), (1, False), (2, False)]
    assert [(i, add) for i, add in P.run_order(d)] == [(r.layer, r.add_embedding) for r in spec.order]
    assert all(r.cache_of is None for r in spec.order)      # every pass keeps its own
    names = model_params(spec)
    for name in ("embed", "head", "final.norm", "final.norm.b", "l0.norm1", "l0.norm1.b", "l0.norm1b", "l0.norm2b.b", "l0.mix.q.conv",
                 "l0.mix.A_log", "l0.mix.dt_bias", "l0.mix.b", "l0.mix.a", "l0.mix.norm", "l0.mlp.router", "l0.mlp.e4.up", "l0.mlp.shared.down",
                 "l1.mix.temp", "l1.mlp.gate", "l2.mix.g", "l2.mix.norm"):
        assert name in names, name
    assert "l2.norm2" not in names and "l0.mlp.e5.up" not in names
    assert names["l0.mix.q.conv"].shape == (32, 3) and names["l0.mix.norm"].shape == (24,) and names["l2.mix.norm"].shape == (48,)
    assert names["l1.mix.temp"].shape == (6,) and names["l0.mlp.router"].shape == (5, 64)
    assert cfg.to_dict()["loop"] == {"start": 0, "stop": 2, "times": 3}
    # without a loop every layer runs once
    d2 = copy.deepcopy(d); del d2["loop"]
    assert [r.layer for r in parse_config(d2)[1].model_spec().order] == [0, 1, 2]


def test_what_the_mixers_ask_of_the_cache():
    from kipp_amd.config import parse_config
    from kipp_amd.parts import part_class
    spec = parse_config(_config())[1].model_spec()
    attention = spec.layers[1].part("mixer")
    need = part_class("mixer", attention.kind).need_of(attention)
    assert (need.num_kv_heads, need.head_dim, need.value_dim, need.window) == (2, 24, 16, 11)
    assert spec.layers[0].part("mixer").channels == 2 * 2 * 16 + 4 * 24
    assert spec.layers[2].block == "sandwich_norm_mixer" and spec.layers[0].block == "sandwich_norm"
    assert spec.layers[0].residual_scale == 0.5


@pytest.mark.parametrize("path, value, text", [
    (("layers", 0, "mixer", "rank"), 3, "rank"),
    (("layers", 1, "mixer", "rot"), {"base": 1.0}, "rot"),
    (("layers", 0, "type"), "mamba", "mamba"),
    (("layers", 1, "mlp", "kind"), "glu", "glu"),
    (("layers", 2, "mixer", "decay"), [0.5], "decay"),
    (("loop", "stop"), 9, "loop"),
    (("layers", 0, "mlp", "router", "top"), 6, "top"),
    (("sliding", ), 4, "sliding"),
])
def test_what_is_not_implemented_is_refused_by_name(path, value, text):
    from kipp_amd.config import ConfigError, parse_config
    d = _config()
    at = d
    for key in path[:-1]:
        at = at[key]
    at[path[-1]] = value
    with pytest.raises(ConfigError, match=text):
        parse_config(d)
