"""Feed-forward parts.  Interface:

    params(spec) -> {local name: ParamSpec}
    load(tensors)
    forward(x, batch) -> delta      x [tokens, hidden] activation type,
                                    delta float32 [tokens, hidden] (or slabs of it,
                                    or a product deferred by `Runtime.linear`)

A feed-forward with `takes_scaled_rows = True` also takes `ScaledRows` for x.
"""
from __future__ import annotations

import torch

from ..runtime import ScaledRows, Weight, WeightedDelta
from .base import ParamSpec, register


@register("feed_forward", "gated_mlp")
class GatedMLP:
    """delta = W_down (silu(W_gate x) * (W_up x))  (/root/reference/src/kipp.c:2633-2653); with `bias_names` every
    projection has a bias: the gate's and the up's are added in the activation's kernel, the down's rides on the delta."""

    graph_safe = True   # forward launches kernels only: no host reads, no data-dependent launches
    takes_scaled_rows = True

    def __init__(self, spec, runtime):
        self.spec = spec
        self.rt = runtime
        self.w_gate_up = self.w_down = None

    @staticmethod
    def params(spec):
        gate, up, down = spec.names
        p = {
            gate: ParamSpec((spec.intermediate_size, spec.hidden_size)),
            up: ParamSpec((spec.intermediate_size, spec.hidden_size)),
            down: ParamSpec((spec.hidden_size, spec.intermediate_size)),
        }
        if getattr(spec, "bias_names", None) is not None:
            for name, width in zip(spec.bias_names, (spec.intermediate_size, spec.intermediate_size, spec.hidden_size)):
                p[name] = ParamSpec((width,), "float", ("normal", 0.1))
        return p

    @staticmethod
    def placement(spec):
        return {name: "float32" for name in (getattr(spec, "bias_names", None) or ())}

    def load(self, tensors):
        gate, up, down = self.spec.names
        g, u = tensors[gate], tensors[up]
        if g.dtype != u.dtype:
            g, u = g.float(), u.float()
        biased = getattr(self.spec, "bias_names", None) is not None
        self.w_gate_up = self.rt.weight(torch.cat([g, u], dim=0).contiguous(), gate_up=self.spec.activation == "silu" and not biased)
        self.w_down = self.rt.weight(tensors[down])
        self.bias_gate_up = self.bias_down = None
        if biased:
            self.bias_gate_up = torch.cat([tensors[self.spec.bias_names[0]], tensors[self.spec.bias_names[1]]]).contiguous()
            self.bias_down = tensors[self.spec.bias_names[2]]

    def forward(self, x, batch=None):
        rt = self.rt
        rows, inner = x.shape[0], self.spec.intermediate_size
        act = rt.empty((rows, inner), rt.act_dtype)
        w = self.w_gate_up
        if self.bias_gate_up is not None:
            # biases: the gate-up product by itself, then the activation's kernel adds them ahead of the activation
            rt.ops.activate(rt.linear(rt.rows_of(x), w, slabs=True), act, self.spec.activation, glu=True, bias=self.bias_gate_up)
            return WeightedDelta.of(rt, rt.linear(act, self.w_down, slabs=True, defer=True), 1.0, self.bias_down)
        if self.spec.activation != "silu":
            # another activation: the gate-up product by itself, then the activation's own kernel (the products that
            # end in the activation are built for silu)
            rt.ops.activate(rt.linear(rt.rows_of(x), Weight(w.rows, None if w.pairs else w.tiles), slabs=True), act, self.spec.activation, glu=True)
            return rt.linear(act, self.w_down, slabs=True, defer=True)
        ours = w.dtype == x.dtype == torch.bfloat16 and rt.streams(rows, x.shape[1], 2 * inner)
        if ours and rows <= rt.few_rows:
            # both products and the activation in one kernel (and the norm's scale, if it was left to us)
            scaled = isinstance(x, ScaledRows)
            # the activation goes to the down projection alone: written in the order that product reads fastest
            major = rt.steps_major_rows and inner % 32 == 0 and rows > 1 and rt._few_rows(rows, inner, self.w_down)
            rt.ops.gemm_skinny_swiglu(x.rows if scaled else x, w.rows, act, tiles=w.tiles,
                                      row_scale=x.scale if scaled else None,
                                      x_steps_major=scaled and x.steps_major, out_steps_major=major)
            return rt.linear(act, self.w_down, slabs=True, defer=True, x_steps_major=major)
        x = rt.rows_of(x)
        if ours and w.pairs and rt.ops.gemm_rows_swiglu_pays(rows, 2 * inner, x.shape[1]):
            # a few dozen rows against a weight with rows enough for every compute unit: the activation at the product's end
            rt.ops.gemm_rows_swiglu(x, w.tiles, act)
        elif ours and w.pairs:
            # streamed from the paired tiles: the columns come out gate tile by gate tile
            rt.ops.swiglu(rt.ops.gemm_rows(x, w.rows, max_parts=12, tiles=w.tiles, pairs=True), act, pairs=True)
        elif w.dtype == x.dtype == torch.bfloat16 and not ours:
            act = rt.gated(x, w, act)       # many rows: both products and the activation, by whichever way is faster
        else:
            rt.ops.swiglu(rt.linear(x, w, slabs=True), act)
        return rt.linear(act, self.w_down, slabs=True, defer=True)


@register("feed_forward", "routed_mlp")
class RoutedMLP:
    """A mixture of experts (`RoutedMLPSpec`): delta = sum over a token's `top` experts of weight_e W_down_e act(W_up_e x),
    plus a shared expert of the same form.  The router's logits come out of a product in float32; choice, sort and the
    experts' products over the sorted rows are kernels whose launches have a fixed shape (the list of row tiles is made on
    the device), so nothing is read back and a step of single tokens can be recorded."""

    graph_safe = True   # forward launches kernels only: no host reads, no data-dependent launches

    def __init__(self, spec, runtime):
        self.spec = spec
        self.rt = runtime
        self.w_router = self.w_up = self.w_down = self.w_shared_up = self.w_shared_down = None

    @staticmethod
    def params(spec):
        s = spec
        up, down = s.names
        p = {s.router_name: ParamSpec((s.experts, s.hidden_size))}
        if getattr(s, "correction_name", None) is not None:
            p[s.correction_name] = ParamSpec((s.experts,), "float", ("normal", 0.1))
        for e in range(s.experts):
            p[s.expert_prefix.format(e) + up] = ParamSpec((s.expert_size, s.hidden_size))
            p[s.expert_prefix.format(e) + down] = ParamSpec((s.hidden_size, s.expert_size))
        if s.shared_size is not None:
            p[s.shared_prefix + up] = ParamSpec((s.shared_size, s.hidden_size))
            p[s.shared_prefix + down] = ParamSpec((s.hidden_size, s.shared_size))
        return p

    @staticmethod
    def placement(spec):
        return {spec.correction_name: "float32"} if getattr(spec, "correction_name", None) is not None else {}

    @staticmethod
    def variants(spec, dtype):
        return [("moe", None)]

    def load(self, tensors):
        s = self.spec
        up, down = s.names
        self.correction = tensors[s.correction_name] if getattr(s, "correction_name", None) is not None else None
        router = tensors[s.router_name]
        pad = -router.shape[0] % 16     # whole tiles of rows for the products
        if pad:
            router = torch.cat([router, torch.zeros((pad, router.shape[1]), dtype=router.dtype, device=router.device)], dim=0)
        self.w_router = self.rt.weight(router.contiguous())
        ups = [tensors[s.expert_prefix.format(e) + up] for e in range(s.experts)]
        downs = [tensors[s.expert_prefix.format(e) + down] for e in range(s.experts)]
        if len({t.dtype for t in ups + downs}) > 1:
            ups, downs = [t.float() for t in ups], [t.float() for t in downs]
        self.w_up = torch.stack(ups).contiguous()           # [experts, inner, hidden]
        self.w_down = torch.stack(downs).contiguous()       # [experts, hidden, inner]
        if s.shared_size is not None:
            self.w_shared_up = self.rt.weight(tensors[s.shared_prefix + up])
            self.w_shared_down = self.rt.weight(tensors[s.shared_prefix + down])

    def forward(self, x, batch=None):
        s, rt, ops = self.spec, self.rt, self.rt.ops
        n = x.shape[0]
        pairs = n * s.top
        dev = rt.device
        z = rt.linear(x, self.w_router, slabs=True)
        chosen = torch.empty((n, s.top), dtype=torch.int32, device=dev)
        weight = rt.empty((n, s.top), torch.float32)
        pair_token = torch.empty((pairs,), dtype=torch.int32, device=dev)
        place = torch.empty((pairs,), dtype=torch.int32, device=dev)
        # bfloat16 experts whose two contractions are multiples of 32 run on the matrix cores, in tiles of 128 rows
        tile_rows = ops.moe_tile_rows(self.w_up.dtype, s.hidden_size, s.expert_size)
        tiles = torch.empty((ops.moe_max_tiles(n, s.experts, s.top, tile_rows), 3), dtype=torch.int32, device=dev)
        if s.router == "sigmoid":
            ops.moe_route(z, s.experts, s.top, s.weight_eps, chosen, weight, pair_token, place, tiles, tile_rows=tile_rows, router="sigmoid",
                          correction=self.correction, groups=s.groups, scale=s.route_scale)
        else:
            ops.moe_route(z, s.experts, s.top, s.weight_eps, chosen, weight, pair_token, place, tiles, tile_rows=tile_rows)
        if x.dtype != self.w_up.dtype:
            x = ops.cast(x, rt.empty(x.shape, self.w_up.dtype))
        inner = ops.moe_expert(x, pair_token, self.w_up, tiles, rt.empty((pairs, s.expert_size), self.w_up.dtype), s.activation, tile_rows=tile_rows)
        y = ops.moe_expert(inner, None, self.w_down, tiles, rt.empty((pairs, s.hidden_size), torch.float32), tile_rows=tile_rows)
        shared = None
        if s.shared_size is not None:
            mid = ops.activate(rt.linear(x, self.w_shared_up, slabs=True), rt.empty((n, s.shared_size), rt.act_dtype), s.activation)
            shared = rt.linear(mid, self.w_shared_down, slabs=True)
        return ops.moe_combine(y, place, weight, shared, rt.empty((n, s.hidden_size), torch.float32))
