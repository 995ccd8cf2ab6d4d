"""Recurrent mixers whose memory is a matrix a head, of fixed size, in the request's slot: linear attention with a fixed
decay a head (`DecayAttentionSpec`), the gated delta rule (`GatedDeltaSpec`) and the selective state space layer in its
dual form (`SSDSpec`).

    decay attention   [q | k | v | gate] = W_in x;  q, k, v through silu;  S_t = a_h S_(t-1) + k_t v_t^T;  o_t = S_t^T q_t
                      delta = W_o (o / rms(o over all heads) * w * sigmoid(gate))
    gated delta       [q | k | v | gate | b | a] = W_in x;  q, k, v through a short causal filter a channel and silu;
                      q, k unit vectors a head (q also over sqrt(d));  beta = sigmoid(b),  g = exp(-exp(A) softplus(a + dt))
                      S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q
                      delta = W_o (o / rms(o) a head * w * silu(gate))
    state space       [z | u | B | C | dt] = W_in x;  u, B, C through a short causal filter a channel (with a bias) and silu;
                      dt = softplus(dt + dt_bias);  S <- exp(-exp(A) dt) S + dt B u^T;  y = S^T C + D u
                      delta = W_o (rms in parts of (y silu(z)) * w)

The recurrences, the gates and the norms run in float32 under either precision; the state is float32.  A prompt portion
walks its tokens in order inside one launch, a single token is a walk of one step of the same kernel, so a position's
result does not depend on how the tokens were cut.
"""
from __future__ import annotations

import torch

from ..cache.needs import StateNeed
from .base import ParamSpec, register


def _stack_rows(rt, rows):
    """The rows of several matrices as one weight, padded to whole tiles of 16 rows."""
    if len({t.dtype for t in rows}) > 1:
        rows = [t.float() for t in rows]
    w = torch.cat(rows, dim=0)
    pad = -w.shape[0] % 16
    if pad:
        w = torch.cat([w, torch.zeros((pad, w.shape[1]), dtype=w.dtype, device=w.device)], dim=0)
    return rt.weight(w.contiguous())


@register("mixer", "decay_attention")
class DecayAttention:
    graph_safe = True   # forward launches kernels only: no host reads, no data-dependent launches

    def __init__(self, spec, runtime):
        self.spec = spec
        self.rt = runtime
        self.w_in = self.w_o = self.norm = self.decays = None

    @staticmethod
    def params(spec):
        s = spec
        q, k, v, g, o, norm = s.names
        hd, hv = s.num_heads * s.head_dim, s.num_heads * s.v_head_dim
        return {q: ParamSpec((hd, s.hidden_size)), k: ParamSpec((hd, s.hidden_size)), v: ParamSpec((hv, s.hidden_size)),
                g: ParamSpec((hv, s.hidden_size)), o: ParamSpec((s.hidden_size, hv)),
                norm: ParamSpec((hv,), "float", ("one_plus_normal", 0.05))}

    @staticmethod
    def placement(spec):
        return {spec.names[5]: "float32"}

    @staticmethod
    def variants(spec, dtype):
        return [("linear_scan", None)]

    def load(self, tensors):
        q, k, v, g, o, norm = self.spec.names
        self.w_in = _stack_rows(self.rt, [tensors[q], tensors[k], tensors[v], tensors[g]])
        self.w_o = self.rt.weight(tensors[o])
        self.norm = tensors[norm]
        self.decays = torch.tensor(self.spec.decays, dtype=torch.float32, device=self.norm.device)

    def cache_need(self):
        return None

    def state_need(self):
        s = self.spec
        return StateNeed((-(-s.num_heads * s.head_dim * s.v_head_dim // 4) * 4,), "float32")

    def forward(self, x, batch, cache, state):
        s, rt, ops = self.spec, self.rt, self.rt.ops
        n = x.shape[0]
        hv = s.num_heads * s.v_head_dim
        proj = rt.linear(x, self.w_in)                    # float32 [n, q | k | v | gate]
        o_raw = rt.empty((n, hv), torch.float32)
        ops.decay_scan(proj, self.decays, state, batch.q_start, batch.q_len, batch.slots, o_raw, s.num_heads, s.head_dim, s.v_head_dim, longest=batch.max_q_len)
        out = ops.scan_finish(o_raw, proj, 2 * s.num_heads * s.head_dim + hv, self.norm, s.norm_eps, "sigmoid", hv, rt.empty((n, hv), rt.act_dtype))
        return rt.linear(out, self.w_o, slabs=True, defer=True)


@register("mixer", "gated_delta")
class GatedDelta:
    graph_safe = True   # forward launches kernels only: no host reads, no data-dependent launches

    def __init__(self, spec, runtime):
        self.spec = spec
        self.rt = runtime
        self.w_in = self.w_o = self.norm = self.conv = self.a_log = self.dt_bias = None

    @staticmethod
    def _names(spec):
        return dict(zip(("q", "k", "v", "q_conv", "k_conv", "v_conv", "b", "a", "a_log", "dt_bias", "gate", "o", "norm"), spec.names))

    @classmethod
    def params(cls, spec):
        n, s = cls._names(spec), spec
        gd, hv = s.num_kv_heads * s.head_dim, s.num_heads * s.v_head_dim
        return {
            n["q"]: ParamSpec((gd, s.hidden_size)), n["k"]: ParamSpec((gd, s.hidden_size)), n["v"]: ParamSpec((hv, s.hidden_size)),
            n["q_conv"]: ParamSpec((gd, s.conv_taps), "float", ("normal", 0.5)), n["k_conv"]: ParamSpec((gd, s.conv_taps), "float", ("normal", 0.5)),
            n["v_conv"]: ParamSpec((hv, s.conv_taps), "float", ("normal", 0.5)),
            n["b"]: ParamSpec((s.num_heads, s.hidden_size)), n["a"]: ParamSpec((s.num_heads, s.hidden_size)),
            n["a_log"]: ParamSpec((s.num_heads,), "float", ("normal", 0.5)), n["dt_bias"]: ParamSpec((s.num_heads,), "float", ("normal", 0.5)),
            n["gate"]: ParamSpec((hv, s.hidden_size)), n["o"]: ParamSpec((s.hidden_size, hv)),
            n["norm"]: ParamSpec((s.v_head_dim,), "float", ("one_plus_normal", 0.05)),
        }

    @classmethod
    def placement(cls, spec):
        n = cls._names(spec)
        return {n[k]: "float32" for k in ("q_conv", "k_conv", "v_conv", "a_log", "dt_bias", "norm")}

    @staticmethod
    def variants(spec, dtype):
        return [("linear_scan", None)]

    def load(self, tensors):
        n = self._names(self.spec)
        self.w_in = _stack_rows(self.rt, [tensors[n[k]] for k in ("q", "k", "v", "gate", "b", "a")])
        self.w_o = self.rt.weight(tensors[n["o"]])
        self.conv = torch.cat([tensors[n[k]] for k in ("q_conv", "k_conv", "v_conv")], dim=0).contiguous()
        self.a_log, self.dt_bias, self.norm = tensors[n["a_log"]], tensors[n["dt_bias"]], tensors[n["norm"]]

    def cache_need(self):
        return None

    def state_need(self):
        s = self.spec
        return StateNeed((self.rt.ops.delta_state_size(s.num_heads, s.num_kv_heads, s.head_dim, s.v_head_dim, s.conv_taps),), "float32")

    def forward(self, x, batch, cache, state):
        s, rt, ops = self.spec, self.rt, self.rt.ops
        n = x.shape[0]
        hv = s.num_heads * s.v_head_dim
        channels = s.channels
        proj = rt.linear(x, self.w_in)                    # float32 [n, q | k | v | gate | b | a]
        prep = rt.empty((n, channels + 2 * s.num_heads), torch.float32)
        ops.delta_prepare(proj, self.conv, self.a_log, self.dt_bias, state, batch.seq_of_token, batch.q_start, batch.q_len, batch.slots, prep,
                          s.num_heads, s.num_kv_heads, s.head_dim, s.v_head_dim, channels + hv, channels + hv + s.num_heads, s.unit_eps)
        o_raw = rt.empty((n, hv), torch.float32)
        ops.delta_scan(prep, state, batch.q_start, batch.q_len, batch.slots, o_raw, s.num_heads, s.num_kv_heads, s.head_dim, s.v_head_dim, longest=batch.max_q_len)
        out = ops.scan_finish(o_raw, proj, channels, self.norm, s.norm_eps, "silu", s.v_head_dim, rt.empty((n, hv), rt.act_dtype))
        return rt.linear(out, self.w_o, slabs=True, defer=True)


@register("mixer", "ssd")
class SSD:
    """The selective state space layer in its dual form (`SSDSpec`): the recurrence is the matrix memories' walk with a
    decay a token and head, keys B and queries C that the heads of a group share, and values dt u."""

    graph_safe = True   # forward launches kernels only: no host reads, no data-dependent launches

    def __init__(self, spec, runtime):
        self.spec = spec
        self.rt = runtime
        self.w_in = self.w_o = self.conv = self.conv_b = self.dt_bias = self.a_log = self.skip = self.norm = None

    @staticmethod
    def _names(spec):
        return dict(zip(("in", "conv", "conv_b", "dt_bias", "a_log", "skip", "norm", "o"), spec.names))

    @classmethod
    def params(cls, spec):
        n, s = cls._names(spec), spec
        return {
            n["in"]: ParamSpec((s.in_dim, s.hidden_size)),
            n["conv"]: ParamSpec((s.channels, s.conv_taps), "float", ("normal", 0.5)),
            n["conv_b"]: ParamSpec((s.channels,), "float", ("normal", 0.1)),
            n["dt_bias"]: ParamSpec((s.num_heads,), "float", ("normal", 0.5)),
            n["a_log"]: ParamSpec((s.num_heads,), "float", ("normal", 0.5)),
            n["skip"]: ParamSpec((s.num_heads,), "float", ("one_plus_normal", 0.2)),
            n["norm"]: ParamSpec((s.inner,), "float", ("one_plus_normal", 0.05)),
            n["o"]: ParamSpec((s.hidden_size, s.inner)),
        }

    @classmethod
    def placement(cls, spec):
        n = cls._names(spec)
        return {n[k]: "float32" for k in ("conv", "conv_b", "dt_bias", "a_log", "skip", "norm")}

    @staticmethod
    def variants(spec, dtype):
        return [("linear_scan", None)]

    def load(self, tensors):
        n = self._names(self.spec)
        self.w_in = _stack_rows(self.rt, [tensors[n["in"]]])
        self.w_o = self.rt.weight(tensors[n["o"]])
        self.conv, self.conv_b = tensors[n["conv"]], tensors[n["conv_b"]]
        self.dt_bias, self.a_log, self.skip, self.norm = tensors[n["dt_bias"]], tensors[n["a_log"]], tensors[n["skip"]], tensors[n["norm"]]

    def cache_need(self):
        return None

    def state_need(self):
        s = self.spec
        return StateNeed((self.rt.ops.ssd_state_size(s.num_heads, s.groups, s.state_size, s.head_dim, s.conv_taps),), "float32")

    def forward(self, x, batch, cache, state):
        s, rt, ops = self.spec, self.rt, self.rt.ops
        n = x.shape[0]
        proj = rt.linear(x, self.w_in)                    # float32 [n, z | u | B | C | dt]
        prep = rt.empty((n, ops.ssd_prep_width(s.num_heads, s.groups, s.state_size, s.head_dim)), torch.float32)
        ops.ssd_prepare(proj, self.conv, self.conv_b, self.a_log, self.dt_bias, state, batch.seq_of_token, batch.q_start, batch.q_len,
                        batch.slots, prep, s.num_heads, s.groups, s.state_size, s.head_dim)
        o_raw = rt.empty((n, s.inner), torch.float32)
        ops.gated_scan(prep, state, batch.q_start, batch.q_len, batch.slots, o_raw, s.num_heads, s.groups, s.state_size, s.head_dim,
                       longest=batch.max_q_len)
        out = ops.ssd_finish(o_raw, prep, 2 * s.groups * s.state_size + s.inner, proj, 0, self.skip, s.head_dim, self.norm, s.norm_eps,
                             s.inner // s.norm_groups, rt.empty((n, s.inner), rt.act_dtype))
        return rt.linear(out, self.w_o, slabs=True, defer=True)
