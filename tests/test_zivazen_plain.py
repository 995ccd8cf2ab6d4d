"""The Zivazen design without a GPU: the plain implementation's mechanisms by hand or against a second formulation, the
configuration's keys and refusals, the tensors the parts declare, what the cache manager is asked for."""
import copy
import math

import numpy as np
import pytest

from tests.plain import zivazen_plain as P


def tiny(name="zivazen-tiny-a"):
    from kipp_amd.config import shape_config
    return shape_config(name)


# =============================================================================== the plain implementation

def test_rotary_frequencies_by_band():
    """A short wavelength is kept, a long one divided by the factor, one in between blended by its place between them."""
    sc = {"factor": 5.0, "low": 1.0, "high": 4.0, "original": 100.0}
    f = P.rotary_frequencies(8, 10000.0, None)
    assert np.allclose(f, [1.0, 0.1, 0.01, 0.001])
    g = P.rotary_frequencies(8, 10000.0, sc)
    # wavelengths 6.28, 62.8, 628, 6283 against 25 and 100
    assert g[0] == f[0] and g[2] == f[2] / 5 and g[3] == f[3] / 5
    s = (100.0 / (2 * math.pi / 0.1) - 1.0) / 3.0
    assert np.isclose(g[1], (1 - s) * 0.1 / 5 + s * 0.1) and f[1] / 5 < g[1] < f[1]


def test_rotation_turns_halves_and_leaves_the_rest():
    x = np.arange(1.0, 7.0).reshape(1, 1, 6)
    out = P.rotate(x, [3], 4, np.array([0.5, 0.25]))
    a, b = 3 * 0.5, 3 * 0.25
    assert np.allclose(out[0, 0], [1 * math.cos(a) - 3 * math.sin(a), 2 * math.cos(b) - 4 * math.sin(b),
                                   3 * math.cos(a) + 1 * math.sin(a), 4 * math.cos(b) + 2 * math.sin(b), 5.0, 6.0])
    assert np.allclose(P.rotate(x, [0], 4, np.array([0.5, 0.25])), x)


def test_sink_and_masks():
    """One added to the denominator: a lone key of score s weighs e^s / (1 + e^s); chunks are counted from position 0."""
    q = np.ones((1, 1, 2))
    k = np.array([[[0.5, 0.5]]])
    v = np.array([[[2.0]]])
    out = P.attention_core(q, k, v, 1.0, lambda i, j: True, sink=True)
    assert np.isclose(out[0, 0, 0], 2.0 * math.e / (1 + math.e))
    assert np.isclose(P.attention_core(q, k, v, 1.0, lambda i, j: True, sink=False)[0, 0, 0], 2.0)
    rng = np.random.default_rng(0)
    t_len = 11
    q, k, v = rng.normal(size=(t_len, 2, 4)), rng.normal(size=(t_len, 1, 4)), rng.normal(size=(t_len, 1, 3))
    size = 4
    out = P.attention_core(q, k, v, 0.7, lambda i, j: i // size == j // size, sink=True)
    for i in (0, 3, 4, 7, 8, 10):
        lo = i - i % size
        s = (q[i, 1] @ k[lo:i + 1, 0].T) * 0.7
        w = np.exp(s) / (1.0 + np.exp(s).sum())
        assert np.allclose(out[i, 1], w @ v[lo:i + 1, 0])


def test_causal_filter_by_hand_and_across_a_cut():
    x = np.array([[1.0, 10.0], [2.0, 20.0], [3.0, 30.0], [4.0, 40.0]])
    w = np.array([[0.5, 1.0, 2.0], [1.0, 0.0, -1.0]])
    b = np.array([0.25, -1.0])
    out = P.causal_filter(x, w, b)
    assert np.allclose(out[0], [2.0 * 1 + 0.25, -10.0 - 1.0])
    assert np.allclose(out[2], [0.5 * 1 + 1.0 * 2 + 2.0 * 3 + 0.25, 10.0 - 30.0 - 1.0])
    again = P.causal_filter(x[2:], w, b, before=x[:2])
    assert np.allclose(again, out[2:])


def test_state_space_walk_against_the_sum_over_earlier_tokens():
    """y_t = sum_{s <= t} (prod_{s < r <= t} a_r) dt_s (C_t . B_s) x_s + D x_t, and a cut with the state handed on."""
    rng = np.random.default_rng(1)
    t_len, heads, p, groups, n = 9, 4, 3, 2, 5
    x, b, c = rng.normal(size=(t_len, heads, p)), rng.normal(size=(t_len, groups, n)), rng.normal(size=(t_len, groups, n))
    dt = P.softplus(rng.normal(size=(t_len, heads)))
    a_log, skip = rng.normal(size=heads) * 0.5, rng.normal(size=heads)
    y, s_end = P.ssd_scan(x, b, c, dt, a_log, skip)
    for h in range(heads):
        g = h // (heads // groups)
        a = np.exp(-np.exp(a_log[h]) * dt[:, h])
        for t in range(t_len):
            ref = skip[h] * x[t, h]
            for s in range(t + 1):
                ref = ref + np.prod(a[s + 1:t + 1]) * dt[s, h] * (c[t, g] @ b[s, g]) * x[s, h]
            assert np.allclose(y[t, h], ref)
    y1, s1 = P.ssd_scan(x[:4], b[:4], c[:4], dt[:4], a_log, skip)
    y2, s2 = P.ssd_scan(x[4:], b[4:], c[4:], dt[4:], a_log, skip, state=s1)
    assert np.allclose(np.concatenate([y1, y2]), y) and np.allclose(s2, s_end)


def test_router_groups_correction_and_weights():
    """The correction moves the choice, not the weights; an expert of a group that does not stay is never chosen, however
    large its score; a group's score is the sum of its two largest; ties go to the lower index."""
    z = np.array([3.0, -3.0, 2.0, 1.9, -0.5, -0.4, -1.0, -1.1])       # groups of two: {0,1} {2,3} {4,5} {6,7}
    s = P.sigmoid(z)
    zero = np.zeros(8)
    chosen, weights, _ = P.route(z, zero, 2, 4, 1, 2.0)
    assert chosen == [2, 3]                                           # group 1: s2 + s3 beats s0 + s1
    assert np.allclose(weights, s[[2, 3]] / s[[2, 3]].sum() * 2.0)
    chosen, _, _ = P.route(z, zero, 2, 4, 2, 1.0)
    assert chosen == [0, 2]                                           # groups 1 and 0 stay; the two largest among them
    corr = np.array([0.0, 0.0, -5.0, -5.0, 0.0, 0.0, 4.0, 4.0])
    chosen, weights, _ = P.route(z, corr, 2, 4, 1, 1.0)
    assert chosen == [6, 7] and np.allclose(weights, s[[6, 7]] / s[[6, 7]].sum())
    chosen, _, _ = P.route(np.zeros(8), zero, 3, 4, 2, 1.0)
    assert chosen == [0, 1, 2]
    chosen, _, _ = P.route(z, np.full(8, -9.0), 2, 4, 1, 1.0)         # negative choice scores: the others count as minus infinity
    assert chosen == [2, 3]


def test_experts_square_their_relu_and_the_gate_comes_before_the_norm():
    w = {"e.up": np.array([[1.0, 0.0], [0.0, 1.0]]), "e.down": np.array([[1.0, 1.0]])}
    assert np.allclose(P.expert_ff(w, "e.", np.array([[3.0, -2.0]])), [[9.0]])
    cfg = tiny("zivazen-tiny-b")
    rng = np.random.default_rng(2)
    m = cfg["layers"][3]["mixer"]["right"]
    heads, p, n, groups, taps = m["heads"], m["vdim"], m["state"], m["groups"], m["conv"]
    inner, width = heads * p, cfg["width"]
    w = {"in": rng.normal(size=(2 * inner + 2 * groups * n + heads, width)) * 0.1, "conv": rng.normal(size=(inner + 2 * groups * n, taps)),
         "conv.b": rng.normal(size=inner + 2 * groups * n) * 0.1, "dt_bias": rng.normal(size=heads), "A_log": rng.normal(size=heads) * 0.3,
         "D": rng.normal(size=heads), "norm": rng.normal(size=inner), "o": np.eye(inner)}
    assert inner == width
    h = rng.normal(size=(6, width))
    out = P.ssd_mixer(cfg, w, "", m, h)
    # the same by hand for the last token's first norm part
    proj = h @ w["in"].T
    z = proj[:, :inner]
    xbc = P.silu(P.causal_filter(proj[:, inner:2 * inner + 2 * groups * n], w["conv"], w["conv.b"]))
    dt = P.softplus(proj[:, -heads:] + w["dt_bias"])
    y, _ = P.ssd_scan(xbc[:, :inner].reshape(6, heads, p), xbc[:, inner:inner + groups * n].reshape(6, groups, n),
                      xbc[:, inner + groups * n:].reshape(6, groups, n), dt, w["A_log"], w["D"])
    gated = y.reshape(6, inner) * P.silu(z)
    part = inner // m["norm_groups"]
    first = gated[-1, :part] / np.sqrt(np.mean(gated[-1, :part] ** 2) + cfg["norm"]["eps"]) * w["norm"][:part]
    assert np.allclose(out[-1, :part], first)


def test_a_changed_token_shows_only_where_the_design_lets_it():
    """In a model of attention layers alone a changed token reaches exactly the positions of its own chunk (the layers
    stack, but a chunk never sees another); with a state space layer it reaches every later position."""
    from kipp_amd.weights.random_init import random_tensor
    from kipp_amd.config import parse_config
    from kipp_amd.engine.model import model_params
    import torch
    cfg = tiny("zivazen-tiny-a")
    only = copy.deepcopy(cfg)
    only["layers"] = [only["layers"][0], only["layers"][2]]
    for variant, reach_all in ((only, False), (cfg, True)):
        spec = parse_config(variant)[1].model_spec()
        w = {name: random_tensor(3, name, p, torch.float32).double().numpy() for name, p in model_params(spec).items()}
        tokens = list(np.random.default_rng(4).integers(0, cfg["vocab"], size=60))
        base = P.forward_whole(variant, w, tokens)
        changed = list(tokens)
        changed[30] = (changed[30] + 1) % cfg["vocab"]
        moved = np.abs(P.forward_whole(variant, w, changed) - base).max(axis=1) > 1e-12
        size = variant["layers"][0]["mixer"]["mask"]["size"]       # 24: the chunk of position 30 is 24 .. 47
        assert not moved[:30].any() and moved[30:48].all()
        assert moved[48:].all() if reach_all else not moved[48:].any()


# =============================================================================== configuration, tensors, cache needs

def test_configuration_keys_and_refusals():
    from kipp_amd.config import ConfigError, parse_config
    cfg = tiny()
    family, typed = parse_config(cfg)
    assert family.name == "Zivazen" and typed.to_dict()["layers"] == cfg["layers"]
    spec = typed.model_spec()
    assert [layer.block for layer in spec.layers] == ["parallel", "parallel", "parallel", "parallel_mixer"]
    first, third = spec.layers[0].part("mixer"), spec.layers[2].part("mixer")
    assert (first.v_mix, third.v_mix) == ("source", "mix") and first.chunk == 24 and first.sink and first.window is None
    assert first.position.kind == "rope_band_scaled" and first.position.rotary_dim == 8
    side = spec.layers[1].part("mixer")
    assert side.kind == "parallel_mixer" and side.left.window == 20 and side.left.position.kind == "rope" and side.right.kind == "ssd"
    assert (side.left_scale, side.right_scale) == (0.9, 1.3)
    routed = spec.layers[1].part("ffn")
    assert routed.router == "sigmoid" and routed.groups == (4, 2) and routed.route_scale == 1.5 and routed.activation == "relu2"
    assert spec.embedding_norm is not None

    def broken(change):
        bad = copy.deepcopy(cfg)
        change(bad)
        with pytest.raises(ConfigError):
            parse_config(bad)
    broken(lambda c: c["layers"][0]["mixer"].update(softcap=3.0))                      # a key the design does not have
    broken(lambda c: c["layers"][0].update(type="lightning"))
    broken(lambda c: c["layers"][1]["mixer"]["right"].update(norm_groups=5))           # does not divide heads * vdim
    broken(lambda c: c["layers"][1]["mlp"]["router"]["groups"].update(count=3))        # 8 experts in 3 groups
    broken(lambda c: c["layers"][1]["mlp"]["router"].update(top=5))                    # more than the kept groups hold
    broken(lambda c: c["layers"][2]["mixer"].update(vdim=16))                          # cannot be mixed with the first layer's values
    broken(lambda c: c["layers"][0]["mixer"]["rot"].update(dims=7))
    broken(lambda c: c["layers"][0]["mixer"]["mask"].update(size=0))
    broken(lambda c: c.update(loop={"start": 0, "stop": 1, "times": 2}))


def test_tensor_names_and_cache_needs():
    from kipp_amd.cache.needs import KVNeed
    from kipp_amd.config import parse_config
    from kipp_amd.engine.model import cache_bytes_per_page, model_params
    spec = parse_config(tiny())[1].model_spec()
    names = model_params(spec)
    for name, shape in (("embed", (160, 64)), ("embed.norm", (64,)), ("l0.norm1", (64,)), ("l0.mix.q.b", (64,)), ("l0.mix.vmix", ()),
                        ("l0.mix.o.b", (64,)), ("l0.mix.q.norm", (16,)), ("l2.mix.vmix", ()), ("l1.mix.left.q", (64, 64)),
                        ("l1.mix.right.in", (2 * 32 + 2 * 32 + 4, 64)), ("l1.mix.right.conv", (96, 4)), ("l1.mix.right.conv.b", (96,)),
                        ("l1.mix.right.A_log", (4,)), ("l1.mix.right.D", (4,)), ("l1.mix.right.norm", (32,)), ("l0.mlp.gate.b", (96,)),
                        ("l0.mlp.down.b", (64,)), ("l1.mlp.router", (8, 64)), ("l1.mlp.correction", (8,)), ("l1.mlp.e7.up", (32, 64)),
                        ("l1.mlp.shared.down", (64, 48)), ("final.norm", (64,)), ("head", (160, 64))):
        assert tuple(names[name].shape) == shape, name
    assert "l1.mix.left.q.b" not in names and "l3.mlp.gate" not in names and "l1.mix.left.q.norm" not in names
    from kipp_amd.parts import part_class
    needs = [part_class("mixer", layer.part("mixer").kind).need_of(layer.part("mixer")) for layer in spec.layers]
    assert needs[0] == KVNeed(2, 16, window=24, v_head_dim=32) and needs[1] == KVNeed(2, 16, window=20, v_head_dim=None)
    assert cache_bytes_per_page(spec, 16, 2) == 16 * 2 * (2 * 2 * (16 + 32) + 2 * 2 * (16 + 16))


def test_plain_runs_a_tiny_model_and_reports_margins():
    from kipp_amd.config import parse_config
    from kipp_amd.engine.model import model_params
    from kipp_amd.weights.random_init import random_tensor
    import torch
    cfg = tiny("zivazen-tiny-b")
    spec = parse_config(cfg)[1].model_spec()
    w = {name: random_tensor(1, name, p, torch.float32).double().numpy() for name, p in model_params(spec).items()}
    layers, margins = [], []
    logits = P.forward_whole(cfg, w, [1, 5, 9, 2, 7], layers, margins)
    assert logits.shape == (5, cfg["vocab"]) and len(layers) == 5 and np.isfinite(logits).all()
    assert len(margins) == 2 * 5 and min(margins) >= 0
