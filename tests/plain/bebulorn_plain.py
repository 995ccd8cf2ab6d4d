"""The plain implementation of the Bebulorn decoder: whole sequences, no cache, no pages, no batching, one
function for each mechanism, NumPy float64.  It shares no code with `kipp_amd`; model folders are read with the
`safetensors` package.

Notation: a sequence has T tokens at positions 0 .. T-1, X [T, width] is the residual stream, E = embed[tokens].

    run order        layers 0 .. start-1 once, then layers start .. stop-1 `times` times over (every pass with memory of
                     its own; X += E in front of every pass after the first), then layers stop ..
    layer            X += m LN_1b(mixer(LN_1(X)));  X += m LN_2b(ff(LN_2(X)))   (m = residual_mult; a layer may have no ff)
    LN(x)            (x - mean x) / sqrt(var x + eps) * w + b
    lightning        q, k, v = silu(Wq h), silu(Wk h), silu(Wv h);  S_t = decay_h S_(t-1) + k_t v_t^T;  o_t = S_t^T q_t;
                     all heads of o side by side over their root mean square, times a weight, times sigmoid(Wg h); Wo
    attention        q, k, v = Wq h, Wk h, Wv h;  every head of v over its own root mean square;
                     s = cap tanh(scale temp_h (q_h . k_g) / cap), g = h // (H / G);  i sees j when 0 <= i - j < size;
                     softmax over the seen keys; Wo
    gated delta      q, k, v = silu(conv(Wq h)), silu(conv(Wk h)), silu(conv(Wv h)), conv a causal filter a channel over
                     the last `taps` inputs; q, k per head over sqrt(sum x^2 + 1e-6), q also times dim^(-1/2);
                     beta = sigmoid(Wb h), g = exp(-exp(A_h) softplus(Wa h + dt_h));
                     S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q;
                     every head of o over its root mean square, times a weight [vdim], times silu(Wg h); Wo
    dense ff         Wd (relu(Wgate h) * (Wup h))
    routed ff        p = softmax(Wr h); the `top` largest p, each over their sum (+ 1e-20), weigh Wd_e gelu(Wu_e h)
                     of their experts; a shared expert of the same form is added for every token
    output           logits = H LN_final(X)
"""
from __future__ import annotations

import json
import math
import os

import numpy as np

DTYPE = np.float64
UNIT_EPS = 1e-6        # inside the root of the unit norm of the delta rule's queries and keys
ROUTE_EPS = 1e-20      # added to the sum of the chosen experts' scores


def linear(x, w):
    return np.asarray(x, dtype=DTYPE) @ np.asarray(w, dtype=DTYPE).T


def sigmoid(z):
    return 1.0 / (1.0 + np.exp(-z))


def silu(z):
    return z * sigmoid(z)


def softplus(z):
    return np.logaddexp(0.0, z)


def gelu_erf(z):
    z = np.asarray(z, dtype=DTYPE)
    return 0.5 * z * (1.0 + np.vectorize(math.erf)(z / math.sqrt(2.0)))


def rms(x, eps):
    """x over its root mean square along the last axis, eps inside the root."""
    x = np.asarray(x, dtype=DTYPE)
    return x / np.sqrt(np.mean(x * x, axis=-1, keepdims=True) + eps)


def layer_norm(x, w, b, eps):
    x = np.asarray(x, dtype=DTYPE)
    mean = x.mean(axis=-1, keepdims=True)
    var = ((x - mean) ** 2).mean(axis=-1, keepdims=True)
    return (x - mean) / np.sqrt(var + eps) * np.asarray(w, dtype=DTYPE) + np.asarray(b, dtype=DTYPE)


def lightning_scan(q, k, v, decay, state=None):
    """q, k [T, H, d], v [T, H, dv], decay [H]: S_t = decay S_(t-1) + k_t v_t^T, o_t = S_t^T q_t.  Returns (o [T, H, dv], S)."""
    t_len, heads, d = q.shape
    dv = v.shape[2]
    s = np.zeros((heads, d, dv), dtype=DTYPE) if state is None else np.array(state, dtype=DTYPE)
    out = np.zeros((t_len, heads, dv), dtype=DTYPE)
    for t in range(t_len):
        for h in range(heads):
            s[h] = decay[h] * s[h] + np.outer(k[t, h], v[t, h])
            out[t, h] = s[h].T @ q[t, h]
    return out, s


def lightning(h, w, p, m, eps):
    """The lightning mixer over a whole sequence; `w` the tensors by file name, `p` the layer's prefix, `m` its sizes."""
    heads, d, dv = m["heads"], m["dim"], m["vdim"]
    t_len = h.shape[0]
    q = silu(linear(h, w[p + "q"])).reshape(t_len, heads, d)
    k = silu(linear(h, w[p + "k"])).reshape(t_len, heads, d)
    v = silu(linear(h, w[p + "v"])).reshape(t_len, heads, dv)
    o, _ = lightning_scan(q, k, v, np.asarray(m["decay"], dtype=DTYPE))
    o = rms(o.reshape(t_len, heads * dv), eps) * np.asarray(w[p + "norm"], dtype=DTYPE)
    return linear(o * sigmoid(linear(h, w[p + "g"])), w[p + "o"])


def window_mask(t_len, size):
    """[i, j] true where position i sees j: 0 <= i - j < size (size None: every j <= i)."""
    i, j = np.arange(t_len)[:, None], np.arange(t_len)[None, :]
    return (j <= i) if size is None else ((j <= i) & (i - j < size))


def capped_attention(q, k, v, groups, scale, temp, cap, size):
    """q [T, H, d], k [T, G, d], v [T, G, dv]; head h reads key/value head h // (H / G)."""
    t_len, heads, _ = q.shape
    mask = window_mask(t_len, size)
    out = np.zeros((t_len, heads, v.shape[2]), dtype=DTYPE)
    for h in range(heads):
        g = h // (heads // groups)
        s = (q[:, h] @ k[:, g].T) * scale * temp[h]
        if cap is not None:
            s = cap * np.tanh(s / cap)
        s = np.where(mask, s, -np.inf)
        e = np.exp(s - s.max(axis=1, keepdims=True))
        out[:, h] = (e / e.sum(axis=1, keepdims=True)) @ v[:, g]
    return out


def attention(h, w, p, m, eps):
    heads, groups, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    t_len = h.shape[0]
    q = linear(h, w[p + "q"]).reshape(t_len, heads, d)
    k = linear(h, w[p + "k"]).reshape(t_len, groups, d)
    v = rms(linear(h, w[p + "v"]).reshape(t_len, groups, dv), eps)
    size = (m.get("mask") or {}).get("size")
    o = capped_attention(q, k, v, groups, m["scale"], np.asarray(w[p + "temp"], dtype=DTYPE), m.get("softcap"), size)
    return linear(o.reshape(t_len, heads * dv), w[p + "o"])


def short_conv(x, taps_w, before=None):
    """y[t, c] = sum_j taps_w[c, j] x[t - (taps - 1) + j, c], zeros (or `before`, the inputs ahead of x) in front."""
    x = np.asarray(x, dtype=DTYPE)
    taps_w = np.asarray(taps_w, dtype=DTYPE)
    taps = taps_w.shape[1]
    front = np.zeros((taps - 1, x.shape[1]), dtype=DTYPE) if before is None else np.asarray(before, dtype=DTYPE)
    padded = np.concatenate([front, x], axis=0)
    out = np.zeros_like(x)
    for j in range(taps):
        out += padded[j:j + x.shape[0]] * taps_w[:, j]
    return out


def unit(x):
    return x / np.sqrt(np.sum(x * x, axis=-1, keepdims=True) + UNIT_EPS)


def delta_scan(q, k, v, beta, g, state=None):
    """q, k [T, H, d] (already unit vectors, q scaled), v [T, H, dv], beta, g [T, H].  Returns (o [T, H, dv], S)."""
    t_len, heads, d = q.shape
    dv = v.shape[2]
    s = np.zeros((heads, d, dv), dtype=DTYPE) if state is None else np.array(state, dtype=DTYPE)
    out = np.zeros((t_len, heads, dv), dtype=DTYPE)
    for t in range(t_len):
        for h in range(heads):
            s[h] = g[t, h] * s[h]
            u = beta[t, h] * (v[t, h] - s[h].T @ k[t, h])
            s[h] = s[h] + np.outer(k[t, h], u)
            out[t, h] = s[h].T @ q[t, h]
    return out, s


def delta(h, w, p, m, eps):
    heads, groups, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    t_len = h.shape[0]
    q = silu(short_conv(linear(h, w[p + "q"]), w[p + "q.conv"])).reshape(t_len, groups, d)
    k = silu(short_conv(linear(h, w[p + "k"]), w[p + "k.conv"])).reshape(t_len, groups, d)
    v = silu(short_conv(linear(h, w[p + "v"]), w[p + "v.conv"])).reshape(t_len, heads, dv)
    q, k = unit(q) * d ** -0.5, unit(k)
    rep = heads // groups
    q, k = np.repeat(q, rep, axis=1), np.repeat(k, rep, axis=1)
    beta = sigmoid(linear(h, w[p + "b"]))
    g = np.exp(-np.exp(np.asarray(w[p + "A_log"], dtype=DTYPE)) * softplus(linear(h, w[p + "a"]) + np.asarray(w[p + "dt_bias"], dtype=DTYPE)))
    o, _ = delta_scan(q, k, v, beta, g)
    o = rms(o, eps) * np.asarray(w[p + "norm"], dtype=DTYPE)
    gate = silu(linear(h, w[p + "g"])).reshape(t_len, heads, dv)
    return linear((o * gate).reshape(t_len, heads * dv), w[p + "o"])


def dense_ff(h, w, p):
    return linear(np.maximum(linear(h, w[p + "gate"]), 0.0) * linear(h, w[p + "up"]), w[p + "down"])


def expert(h, w, p):
    return linear(gelu_erf(linear(h, w[p + "up"])), w[p + "down"])


ROUTE_MARGINS = None     # a list, when someone wants them: every call of `route` appends its tokens' margins [T]


def route(h, w_router, top):
    """(chosen experts [T, top], their weights [T, top]).  A token's margin is the gap between the logit of its last
    chosen expert and the largest one left out: where it is small, reduced precision may choose otherwise."""
    z = linear(h, w_router)
    if ROUTE_MARGINS is not None:
        ordered = -np.sort(-z, axis=1)
        ROUTE_MARGINS.append(ordered[:, top - 1] - ordered[:, top] if top < z.shape[1] else np.full(z.shape[0], np.inf))
    e = np.exp(z - z.max(axis=1, keepdims=True))
    s = e / e.sum(axis=1, keepdims=True)
    chosen = np.argsort(-s, axis=1, kind="stable")[:, :top]
    picked = np.take_along_axis(s, chosen, axis=1)
    return chosen, picked / (picked.sum(axis=1, keepdims=True) + ROUTE_EPS)


def routed_ff(h, w, p, mlp):
    chosen, weights = route(h, w[p + "router"], mlp["router"]["top"])
    out = np.zeros((h.shape[0], np.asarray(w[p + "e0.down"]).shape[0]), dtype=DTYPE)
    for t in range(h.shape[0]):
        for e, a in zip(chosen[t], weights[t]):
            out[t] += a * expert(h[t:t + 1], w, f"{p}e{e}.")[0]
    if mlp.get("shared") is not None:
        out += expert(h, w, p + "shared.")
    return out


MIXERS = {"lightning": lightning, "attention": attention, "delta": delta}


def run_order(config):
    """Layer indices in the order they run, and for each run whether the embedding is added in front of it."""
    n = len(config["layers"])
    loop = config.get("loop")
    if not loop:
        return [(i, False) for i in range(n)]
    start, stop, times = loop["start"], loop["stop"], loop["times"]
    order = [(i, False) for i in range(start)]
    for rep in range(times):
        order += [(i, rep > 0 and i == start) for i in range(start, stop)]
    return order + [(i, False) for i in range(stop, n)]


def forward_whole(config, w, tokens, return_layers=False):
    """float64 logits [T, vocab] of a whole sequence (and, on request, the residual stream after every run)."""
    eps, m = config["norm"]["eps"], config["residual_mult"]
    e = np.asarray(w["embed"], dtype=DTYPE)[np.asarray(tokens)]
    x = e.copy()
    kept = []
    for i, add_e in run_order(config):
        layer = config["layers"][i]
        p = f"l{i}."
        if add_e:
            x = x + e
        h = layer_norm(x, w[p + "norm1"], w[p + "norm1.b"], eps)
        y = MIXERS[layer["type"]](h, w, p + "mix.", layer["mixer"], eps)
        x = x + m * layer_norm(y, w[p + "norm1b"], w[p + "norm1b.b"], eps)
        mlp = layer.get("mlp")
        if mlp is not None:
            h = layer_norm(x, w[p + "norm2"], w[p + "norm2.b"], eps)
            y = dense_ff(h, w, p + "mlp.") if mlp["kind"] == "dense" else routed_ff(h, w, p + "mlp.", mlp)
            x = x + m * layer_norm(y, w[p + "norm2b"], w[p + "norm2b.b"], eps)
        kept.append(x.copy())
    logits = linear(layer_norm(x, w["final.norm"], w["final.norm.b"], eps), w["head"])
    return (logits, np.stack(kept)) if return_layers else logits


def load_folder(model_dir):
    """(config dict, {name: float64 array}) of a model folder."""
    import torch
    from safetensors import safe_open
    with open(os.path.join(model_dir, "config.json"), "r", encoding="utf-8") as f:
        config = json.load(f)
    weights = {}
    with safe_open(os.path.join(model_dir, "model.safetensors"), framework="pt") as f:
        for name in f.keys():
            weights[name] = f.get_tensor(name).to(torch.float64).numpy()
    return config, weights
