"""The plain implementation of the Zivazen decoder: whole sequences, no cache, no pages, no batching, one function
for each mechanism, NumPy float64.  It shares no code with `kipp_amd`; model folders are read with the `safetensors`
package.

Notation: a sequence has T tokens at positions 0 .. T-1, X [T, width] is the residual stream, N(x; w) = x / sqrt(mean
x^2 + eps) * w.

    input            X = N(embed[tokens]; embed.norm)
    layer            h = N(X; norm1);  X += mixer(h) + ff(h)            (a layer may have no ff)
    attention        q, k, v = Wq h + bq, Wk h + bk, Wv h + bv;  q, k a head through N(.; q.norm), N(.; k.norm);
                     the first `dims` numbers of every q and k head turned by the position (halves paired, frequencies
                     stretched for long contexts);  s_ij = scale q_i . k_j for j <= i in i's chunk (floor(i / size) =
                     floor(j / size));  p_ij = e^s_ij / (1 + sum_j e^s_ij);  o_i = sum_j p_ij v_j;  Wo o + bo.
                     Value mixing: the first layer that mixes keeps its v; every later one uses (1 - lam) v + lam v_first
    parallel         left_scale * window_attention(h) + right_scale * ssd(h)
      left           q, k, v = Wq h, Wk h, Wv h;  rotation as above (no stretching unless given);  i sees j when
                     0 <= i - j < size;  softmax;  Wo
      right          [z | x | B | C | dt] = W_in h;  x, B, C through a causal filter a channel (with bias) and silu;
                     dt = softplus(dt + dt_bias);  S_t = exp(-exp(A_h) dt) S_(t-1) + dt B_t x_t^T;  y_t = S_t^T C_t + D_h x_t;
                     y * silu(z), then N in `norm_groups` equal parts (times .norm), then Wo
    dense ff         Wd (silu(Wg h + bg) * (Wu h + bu)) + bd
    routed ff        s = sigmoid(Wr h); choice scores c = s + correction; experts in `count` groups of neighbours, a
                     group's score the sum of its two largest c, only the `keep` best groups stay; the `top` largest c
                     among them are chosen; weights s / (sum of the chosen s + 1e-20) * router scale;
                     sum of weight_e Wd_e relu(Wu_e h)^2, plus a shared expert of the same form for every token
    output           logits = head N(X; final.norm)
"""
from __future__ import annotations

import json
import math
import os

import numpy as np

DTYPE = np.float64
ROUTE_EPS = 1e-20


def linear(x, w, b=None):
    y = np.asarray(x, dtype=DTYPE) @ np.asarray(w, dtype=DTYPE).T
    return y if b is None else y + np.asarray(b, dtype=DTYPE)


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return np.logaddexp(0.0, z)


def rms_norm(x, w, eps):
    x = np.asarray(x, dtype=DTYPE)
    y = x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)
    return y if w is None else y * np.asarray(w, dtype=DTYPE)


def rotary_frequencies(dims, base, scaling=None):
    """f_i = base^(-2i / dims), i < dims / 2; with `scaling` (factor, low, high, original) a frequency whose wavelength is
    longer than original / low is divided by factor, one shorter than original / high is kept, and between the two the
    divided and the kept frequency are blended linearly in original / wavelength."""
    f = np.array([float(base) ** (-2.0 * i / dims) for i in range(dims // 2)], dtype=DTYPE)
    if scaling is None:
        return f
    factor, low, high, original = (float(scaling[k]) for k in ("factor", "low", "high", "original"))
    out = f.copy()
    for i, fi in enumerate(f):
        wavelength = 2.0 * math.pi / fi
        if wavelength < original / high:
            continue
        if wavelength > original / low:
            out[i] = fi / factor
        else:
            s = (original / wavelength - low) / (high - low)
            out[i] = (1.0 - s) * fi / factor + s * fi
    return out


def rotate(x, positions, dims, freq):
    """x [T, heads, d]: the first `dims` numbers of every head turned, number i paired with number i + dims / 2."""
    x = np.array(x, dtype=DTYPE)
    half = dims // 2
    angle = np.asarray(positions, dtype=DTYPE)[:, None] * freq[None, :]        # [T, half]
    cos, sin = np.cos(angle)[:, None, :], np.sin(angle)[:, None, :]
    u, v = x[..., :half].copy(), x[..., half:dims].copy()
    x[..., :half] = u * cos - v * sin
    x[..., half:dims] = v * cos + u * sin
    return x


def attention_core(q, k, v, scale, visible, sink):
    """q [T, H, d], k [T, G, d], v [T, G, dv]; visible(i, j) for j <= i; `sink` adds one to the softmax's denominator."""
    t_len, heads, _ = q.shape
    rep = heads // k.shape[1]
    out = np.zeros((t_len, heads, v.shape[2]), dtype=DTYPE)
    for i in range(t_len):
        js = [j for j in range(i + 1) if visible(i, j)]
        for h in range(heads):
            g = h // rep
            s = np.array([np.dot(q[i, h], k[j, g]) for j in js], dtype=DTYPE) * scale
            m = max(s.max(), 0.0) if sink else s.max()
            e = np.exp(s - m)
            denom = e.sum() + (math.exp(-m) if sink else 0.0)
            p = e / denom
            out[i, h] = sum(p[n] * v[j, g] for n, j in enumerate(js))
    return out


def chunk_attention(cfg, w, prefix, m, h, positions, v_first):
    """The attention mixer.  Returns (result, the values a later mixing layer reads)."""
    eps = cfg["norm"]["eps"]
    t_len = h.shape[0]
    heads, groups, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = linear(h, w[prefix + "q"], w[prefix + "q.b"]).reshape(t_len, heads, d)
    k = linear(h, w[prefix + "k"], w[prefix + "k.b"]).reshape(t_len, groups, d)
    v = linear(h, w[prefix + "v"], w[prefix + "v.b"]).reshape(t_len, groups, dv)
    q = rms_norm(q, w[prefix + "q.norm"], eps)
    k = rms_norm(k, w[prefix + "k.norm"], eps)
    rot = m["rot"]
    freq = rotary_frequencies(rot["dims"], rot["base"], rot.get("scaling"))
    q, k = rotate(q, positions, rot["dims"], freq), rotate(k, positions, rot["dims"], freq)
    keep = v_first
    if m.get("v_mix"):
        if v_first is None:
            keep = v
        else:
            lam = float(np.asarray(w[prefix + "vmix"], dtype=DTYPE))
            v = (1.0 - lam) * v + lam * v_first
    size = (m.get("mask") or {}).get("size")        # no mask: every earlier position is seen
    o = attention_core(q, k, v, m["scale"], lambda i, j: size is None or positions[i] // size == positions[j] // size, sink=True)
    return linear(o.reshape(t_len, heads * dv), w[prefix + "o"], w[prefix + "o.b"]), keep


def window_attention(w, prefix, m, h, positions):
    t_len = h.shape[0]
    heads, groups, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    q = linear(h, w[prefix + "q"]).reshape(t_len, heads, d)
    k = linear(h, w[prefix + "k"]).reshape(t_len, groups, d)
    v = linear(h, w[prefix + "v"]).reshape(t_len, groups, dv)
    rot = m["rot"]
    freq = rotary_frequencies(rot["dims"], rot["base"], rot.get("scaling"))
    q, k = rotate(q, positions, rot["dims"], freq), rotate(k, positions, rot["dims"], freq)
    size = (m.get("mask") or {}).get("size")
    o = attention_core(q, k, v, m["scale"], lambda i, j: size is None or positions[i] - positions[j] < size, sink=False)
    return linear(o.reshape(t_len, heads * dv), w[prefix + "o"])


def causal_filter(x, taps_w, bias, before=None):
    """x [T, C], taps_w [C, taps] (the last column weighs the current token's input), zeros (or `before`
    [taps - 1, C]) ahead of the first token."""
    x = np.asarray(x, dtype=DTYPE)
    taps_w = np.asarray(taps_w, dtype=DTYPE)
    taps = taps_w.shape[1]
    ahead = np.zeros((taps - 1, x.shape[1]), dtype=DTYPE) if before is None else np.asarray(before, dtype=DTYPE)
    full = np.concatenate([ahead, x], axis=0)
    out = np.zeros_like(x)
    for t in range(x.shape[0]):
        for j in range(taps):
            out[t] += taps_w[:, j] * full[t + j]
    return out + np.asarray(bias, dtype=DTYPE)


def ssd_scan(x, b, c, dt, a_log, d_skip, state=None):
    """x [T, H, P], b and c [T, G, N], dt [T, H] (after softplus): S_t = exp(-exp(A_h) dt) S_(t-1) + dt B_t x_t^T,
    y_t = S_t^T C_t + D_h x_t.  Returns (y [T, H, P], S [H, N, P])."""
    t_len, heads, p = x.shape
    groups, n = b.shape[1], b.shape[2]
    rep = heads // groups
    s = np.zeros((heads, n, p), dtype=DTYPE) if state is None else np.array(state, dtype=DTYPE)
    y = np.zeros((t_len, heads, p), dtype=DTYPE)
    for t in range(t_len):
        for h in range(heads):
            g = h // rep
            s[h] = math.exp(-math.exp(a_log[h]) * dt[t, h]) * s[h] + dt[t, h] * np.outer(b[t, g], x[t, h])
            y[t, h] = s[h].T @ c[t, g] + d_skip[h] * x[t, h]
    return y, s


def ssd_mixer(cfg, w, prefix, m, h):
    eps = cfg["norm"]["eps"]
    t_len = h.shape[0]
    heads, p, n, groups = m["heads"], m["vdim"], m["state"], m["groups"]
    inner = heads * p
    proj = linear(h, w[prefix + "in"])
    z, xbc, dt = proj[:, :inner], proj[:, inner:2 * inner + 2 * groups * n], proj[:, 2 * inner + 2 * groups * n:]
    assert dt.shape[1] == heads
    xbc = silu(causal_filter(xbc, w[prefix + "conv"], w[prefix + "conv.b"]))
    x = xbc[:, :inner].reshape(t_len, heads, p)
    b = xbc[:, inner:inner + groups * n].reshape(t_len, groups, n)
    c = xbc[:, inner + groups * n:].reshape(t_len, groups, n)
    dt = softplus(dt + np.asarray(w[prefix + "dt_bias"], dtype=DTYPE))
    y, _ = ssd_scan(x, b, c, dt, np.asarray(w[prefix + "A_log"], dtype=DTYPE), np.asarray(w[prefix + "D"], dtype=DTYPE))
    y = y.reshape(t_len, inner) * silu(z)
    parts = m["norm_groups"]
    y = rms_norm(y.reshape(t_len, parts, inner // parts), None, eps).reshape(t_len, inner) * np.asarray(w[prefix + "norm"], dtype=DTYPE)
    return linear(y, w[prefix + "o"])


def dense_ff(w, prefix, h):
    gate = linear(h, w[prefix + "gate"], w[prefix + "gate.b"])
    up = linear(h, w[prefix + "up"], w[prefix + "up.b"])
    return linear(silu(gate) * up, w[prefix + "down"], w[prefix + "down.b"])


def route(z, correction, top, group_count, group_keep, scale):
    """z [E] router logits of one token -> (chosen experts, their weights, the margin of the choice)."""
    s = sigmoid(np.asarray(z, dtype=DTYPE))
    c = s + np.asarray(correction, dtype=DTYPE)
    experts = len(s)
    size = experts // group_count
    group_score = np.array([np.sort(c[g * size:(g + 1) * size])[-2:].sum() if size > 1 else c[g * size]
                            for g in range(group_count)])
    order = sorted(range(group_count), key=lambda g: (-group_score[g], g))
    kept = set(order[:group_keep])
    masked = np.array([c[e] if e // size in kept else -np.inf for e in range(experts)])
    ranked = sorted(range(experts), key=lambda e: (-masked[e], e))
    chosen = ranked[:top]
    weights = s[chosen] / (s[chosen].sum() + ROUTE_EPS) * scale
    margin = masked[ranked[top - 1]] - masked[ranked[top]] if top < experts else np.inf
    if group_keep < group_count:
        margin = min(margin, group_score[order[group_keep - 1]] - group_score[order[group_keep]])
    return chosen, weights, margin


def expert_ff(w, prefix, h):
    return linear(np.maximum(linear(h, w[prefix + "up"]), 0.0) ** 2, w[prefix + "down"])


def routed_ff(w, prefix, mlp, h, margins=None):
    r = mlp["router"]
    groups = r.get("groups") or {"count": 1, "keep": 1}
    z = linear(h, w[prefix + "router"])
    out = np.zeros_like(h, dtype=DTYPE)
    for t in range(h.shape[0]):
        chosen, weights, margin = route(z[t], w[prefix + "correction"], r["top"], groups["count"], groups["keep"], r.get("scale", 1.0))
        if margins is not None:
            margins.append(margin)
        for e, wt in zip(chosen, weights):
            out[t] += wt * expert_ff(w, f"{prefix}e{e}.", h[t:t + 1])[0]
    if mlp.get("shared") is not None:
        out += expert_ff(w, prefix + "shared.", h)
    return out


def forward_whole(cfg, w, tokens, layers_out=None, margins=None):
    """Logits [T, vocab] of a whole sequence.  `layers_out`: a list that receives X after every layer."""
    eps = cfg["norm"]["eps"]
    positions = list(range(len(tokens)))
    x = rms_norm(np.asarray(w["embed"], dtype=DTYPE)[list(tokens)], w["embed.norm"], eps)
    v_first = None
    for i, layer in enumerate(cfg["layers"]):
        h = rms_norm(x, w[f"l{i}.norm1"], eps)
        m = layer["mixer"]
        if layer["type"] == "attention":
            delta, v_first = chunk_attention(cfg, w, f"l{i}.mix.", m, h, positions, v_first)
        elif layer["type"] == "parallel":
            delta = m["left_scale"] * window_attention(w, f"l{i}.mix.left.", m["left"], h, positions) \
                + m["right_scale"] * ssd_mixer(cfg, w, f"l{i}.mix.right.", m["right"], h)
        else:
            raise ValueError(f"layer type {layer['type']!r}")
        mlp = layer.get("mlp")
        if mlp is not None:
            if mlp["kind"] == "dense":
                delta = delta + dense_ff(w, f"l{i}.mlp.", h)
            elif mlp["kind"] == "moe":
                delta = delta + routed_ff(w, f"l{i}.mlp.", mlp, h, margins)
            else:
                raise ValueError(f"feed-forward kind {mlp['kind']!r}")
        x = x + delta
        if layers_out is not None:
            layers_out.append(x.copy())
    return linear(rms_norm(x, w["final.norm"], eps), w["head"])


def load_folder(folder):
    """(config dict, {name: float64 array}) of a model folder."""
    import torch
    from safetensors.torch import load_file
    with open(os.path.join(folder, "config.json")) as f:
        cfg = json.load(f)
    tensors = load_file(os.path.join(folder, "model.safetensors"))
    return cfg, {k: v.to(torch.float64).numpy() for k, v in tensors.items()}
