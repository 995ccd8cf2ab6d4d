"""Token mixers.  Interface of a mixer:

    params(spec) -> {local name: ParamSpec}
    load(tensors)
    cache_need() -> KVNeed or None      what it keeps per token, in pages
    state_need() -> StateNeed or None   what it keeps per request, of fixed size
    forward(x, batch, cache, state) -> delta
        x      [tokens, hidden] in the activation type (the normed residual)
        batch  the step's StepBatch (positions, sequence of each token, tables)
        cache  the KVCacheView of this run (None if cache_need() is None)
        state  tensor [slots, ...] of this run (None if state_need() is None)
        delta  float32 [tokens, hidden], added to the residual by the block
               (or slabs of it, or a product deferred by `Runtime.linear`)

A mixer with `takes_scaled_rows = True` passes x on to `Runtime.linear` only,
which also takes rows whose norm scale is still to be applied.
"""
from __future__ import annotations

import math

import torch

from ..cache.needs import KVNeed
from .base import ParamSpec, build_part, register



@register("mixer", "attention")
class Attention:
    """Causal grouped-query attention with optional per-head q/k RMSNorm, a
    rotary position part and an optional window, over the paged cache
    (/root/reference/src/kipp.c:2950-2993).  Query head h reads key/value head
    h // (n_q / n_kv)."""

    graph_safe = True   # forward launches kernels only: no host reads, no data-dependent launches
    takes_scaled_rows = True

    def __init__(self, spec, runtime):
        self.spec = spec
        self.rt = runtime
        self.position = build_part("position", spec.position, runtime)
        self.scale = spec.scale if spec.scale is not None else 1.0 / math.sqrt(spec.head_dim)
        self.w_qkv = self.w_o = self.q_norm = self.k_norm = None
        # Values narrower than their keys under bfloat16: a value's row in the cache is as wide as a key's, the rest zeros,
        # so that the matrix-core kernels (which take one head size) run; the output projection gets zero columns to match
        # (a mixer that reads another run's cache finds that run's rows, padded or not)
        self.pad_values = runtime.dtype == "bfloat16" and spec.value_dim < spec.head_dim and spec.head_dim % 16 == 0 \
            and spec.num_heads // spec.num_kv_heads <= 16 and not (spec.sink and spec.chunk is None and spec.window is None)
        self.w_o_padded = None

    @staticmethod
    def params(spec):
        q, k, v, o, q_norm, k_norm = spec.names
        p = {q: ParamSpec((spec.q_dim, spec.hidden_size)), o: ParamSpec((spec.hidden_size, spec.out_dim))}
        if spec.own_kv:
            p[k] = ParamSpec((spec.kv_dim, spec.hidden_size))
            p[v] = ParamSpec((spec.v_dim, spec.hidden_size))
        if spec.bias:
            for name, width in zip(spec.bias_names, (spec.q_dim, spec.kv_dim, spec.v_dim)):
                if spec.own_kv or name == spec.bias_names[0]:
                    p[name] = ParamSpec((width,), "float", ("normal", 0.1))
        if spec.qk_norm_eps is not None and spec.qk_norm_weight:
            p[q_norm] = ParamSpec((spec.head_dim,), "float", ("one_plus_normal", 0.05))
            p[k_norm] = ParamSpec((spec.head_dim,), "float", ("one_plus_normal", 0.05))
        if spec.head_temp is not None:
            p[spec.head_temp] = ParamSpec((spec.num_heads,), "float", ("one_plus_normal", 0.2))
        if spec.out_bias is not None:
            p[spec.out_bias] = ParamSpec((spec.hidden_size,), "float", ("normal", 0.1))
        if spec.v_mix is not None:
            p[spec.v_mix_name] = ParamSpec((), "float", ("abs_normal", 0.3))
        return p

    @staticmethod
    def placement(spec):
        """What enters norms and sums in float32 is widened on the device (exact)."""
        return {name: "float32" for name in spec.names[4:] + tuple(spec.bias_names) + ((spec.head_temp,) if spec.head_temp else ())
                + ((spec.out_bias,) if spec.out_bias else ()) + ((spec.v_mix_name,) if spec.v_mix else ())}

    @staticmethod
    def variants(spec, dtype):
        """The builds of its specialised kernels (one per head size; decode also per number of query heads
        that share a key/value head).  Under float32, and for more than 16 heads a group, the generic
        attention kernel runs, which every model has."""
        out = [("rope_kv", None) if spec.plain else ("head_prepare", None), ("attention_generic", None)]
        if not spec.plain and getattr(spec.position, "kind", "none") != "none":
            out.append(("rope_kv", None))       # the step's table of angles
        if dtype != "bfloat16" or spec.head_dim % 16 or spec.value_dim > spec.head_dim or (spec.sink and spec.chunk is None and spec.window is None):
            return out      # (values narrower than their keys are cached in rows as wide as the keys: the same builds)
        from ..csrc.ops import attention_build_defines
        group = spec.num_heads // spec.num_kv_heads
        # capped scores, chunks and the added one in the denominator: builds of their own
        extras = (spec.softcap is not None, spec.chunk is not None, spec.sink)
        out.append(("attention_prefill", attention_build_defines(spec.head_dim, None, *extras)))
        if group <= 16:
            out.append(("attention_decode", attention_build_defines(spec.head_dim, group, *extras)))
        return out

    def load(self, tensors):
        import torch
        s = self.spec
        names = s.names
        rows = [tensors[names[0]]] + ([tensors[names[1]], tensors[names[2]]] if s.own_kv else [])
        if len({t.dtype for t in rows}) > 1:
            rows = [t.float() for t in rows]
        # rows concatenated: one product serves q, k and v; no output element changes
        self.w_qkv = self.rt.weight(torch.cat(rows, dim=0).contiguous())
        self.w_o = self.rt.weight(tensors[names[3]])
        if self.pad_values:
            w = tensors[names[3]].reshape(s.hidden_size, s.num_heads, s.value_dim)
            wide = torch.zeros((s.hidden_size, s.num_heads, s.head_dim), dtype=w.dtype, device=w.device)
            wide[:, :, :s.value_dim] = w
            self.w_o_padded = self.rt.weight(wide.reshape(s.hidden_size, s.num_heads * s.head_dim).contiguous())
        if s.qk_norm_eps is not None and s.qk_norm_weight:
            self.q_norm = tensors[names[4]]
            self.k_norm = tensors[names[5]]
        self.head_temp = tensors[s.head_temp] if s.head_temp is not None else None
        self.head_temp_capped = None
        if s.softcap is not None:
            # for the matrix-core kernels, which cap what they are given: queries times (scale / cap) beside the head's factor
            ones = torch.ones(s.num_heads, dtype=torch.float32, device=self.w_o.rows.device)
            self.head_temp_capped = ((self.head_temp.float() if self.head_temp is not None else ones) * (self.scale / s.softcap)).contiguous()
        self.bias = None
        if s.bias:
            held = [tensors[name] for name in (s.bias_names if s.own_kv else s.bias_names[:1])]
            if not s.own_kv:        # the kernel's bias runs over q | k | v: nothing is added where nothing is written
                held.append(torch.zeros(s.kv_dim + s.v_dim, dtype=torch.float32, device=held[0].device))
            self.bias = torch.cat([t.float() for t in held]).contiguous()
        self.out_bias = tensors[s.out_bias] if s.out_bias is not None else None
        self.v_lambda = tensors[s.v_mix_name].reshape(1).contiguous() if s.v_mix == "mix" else None

    @staticmethod
    def need_of(spec):
        """What a mixer of this spec keeps per token, known without building it."""
        # a chunk never reads further back than its own length: for the pages it is a window of that size
        return KVNeed(num_kv_heads=spec.num_kv_heads, head_dim=spec.head_dim, window=spec.window if spec.chunk is None else spec.chunk,
                      page_size=spec.page_size, v_head_dim=spec.v_head_dim)

    def cache_need(self):
        need = self.need_of(self.spec)
        if self.pad_values:
            need = KVNeed(num_kv_heads=need.num_kv_heads, head_dim=need.head_dim, window=need.window, page_size=need.page_size,
                          v_head_dim=None, keep_first=need.keep_first)
        return need

    def state_need(self):
        return None

    def forward(self, x, batch, cache, state=None):
        s, rt = self.spec, self.rt
        n = x.shape[0]
        if not s.plain:
            return self._forward_prepared(x, batch, cache)
        inv_freq, rotary_dim = self.position.rotary_table()
        angles = self.position.angles(batch) if hasattr(self.position, "angles") and hasattr(batch, "step_cache") else None
        table = batch.block_tables[cache.group]
        eps = s.qk_norm_eps if s.qk_norm_eps is not None else 0.0
        pairing = getattr(self.position, "pairing", "half")
        # a table row is as wide as the longest context of this step, so what decides is what the step needs
        fast = rt.dtype == "bfloat16" and s.head_dim % 16 == 0 \
            and rt.ops.attention_fast_ok(s.num_heads, s.num_kv_heads, cache.page_size, table.shape[1])
        if rt.dtype == "bfloat16" and not fast:
            rt.generic_attention_launches += 1      # the slow kernel class: a measurement must know it ran
        # single tokens only: norm, rotation, cache write and attention in one kernel, for a few of them (with
        # more rows or long contexts every split's workgroup would prepare the queries again, which costs more
        # than the rotary kernel it saves) and wherever the kernel that walks whole contexts or long ranges runs
        fused = fast and not batch.n_portions and batch.n_decode == n and pairing == "half" \
            and rt.ops.attention_decode_fused_ok(s.head_dim, rotary_dim, inv_freq is not None) \
            and ((n <= rt.fused_decode_rows and batch.max_decode_ctx < rt.fused_decode_keys)
                 or rt.ops.attention_decode_streams(n, s.num_kv_heads, s.head_dim, s.num_heads // s.num_kv_heads,
                                                    cache.page_size, batch.max_decode_ctx, s.window or 0))
        qkv = rt.linear(x, self.w_qkv, slabs=rt.ops.DECODE_FUSED_SLABS if fused else True)
        if fused:
            out = rt.empty((n, s.q_dim), rt.act_dtype)
            # the mixed heads go to the output projection alone: in the order that product reads fastest, if it is a few-rows one
            major = rt.steps_major_rows and n > 1 and rt._few_rows(n, s.q_dim, self.w_o)
            rt.ops.attention_decode_fused(qkv, cache.k, cache.v, out, batch.decode_rows, batch.positions,
                                          batch.seq_of_token, table, s.num_heads, s.num_kv_heads, s.head_dim,
                                          self.q_norm, self.k_norm, eps, inv_freq, rotary_dim, cache.writable,
                                          self.scale, s.window or 0, batch.max_decode_ctx, self._workspace(batch),
                                          angles=angles, out_steps_major=major)
            return rt.linear(out, self.w_o, slabs=True, defer=True, x_steps_major=major)
        q = rt.ops.qk_norm_rope_kv_write(
            qkv, rt.empty((n, s.q_dim), rt.act_dtype), cache.k, cache.v,
            batch.positions, batch.seq_of_token, table, s.num_heads, s.num_kv_heads, s.head_dim,
            self.q_norm, self.k_norm, eps, inv_freq, rotary_dim, write_kv=cache.writable, angles=angles, pairing=pairing)
        out = rt.empty((n, s.q_dim), rt.act_dtype)
        paged_attention(rt, batch, q, out, cache.k, cache.v, cache.page_size, table, s.num_heads, s.num_kv_heads, s.head_dim,
                        s.head_dim, self.scale, s.window, fast, owner=self)
        return rt.linear(out, self.w_o, slabs=True, defer=True)

    def _prefill_work(self, batch):
        """The prefill kernel's work list for this mixer's sizes (`prefill_work`)."""
        return prefill_work(self.rt, batch, self.spec.num_heads, self.spec.head_dim, self.spec.chunk or self.spec.window)

    def _workspace(self, batch):
        """The split decode kernel's partial results for this mixer's sizes (`decode_workspace`)."""
        return decode_workspace(self.rt, batch, self.spec.num_heads, self.spec.head_dim)

    def _forward_prepared(self, x, batch, cache):
        """The mixer with any of: biases, a norm without weights, a factor on the queries that grows with the position,
        values of their own width, keys and values of another run, chunks, the added one in the softmax's denominator,
        values mixed with an earlier run's, a bias on the output.  One kernel makes the heads ready from the input product
        (and turns them, where the mixer rotates); the attention kernels are the same."""
        s, rt = self.spec, self.rt
        from ..runtime import WeightedDelta
        inv_freq, rotary_dim = self.position.rotary_table()
        angles = None
        if inv_freq is not None:
            if getattr(self.position, "pairing", "half") != "half":
                raise NotImplementedError("the kernel that makes these heads ready turns halves of a head, not neighbours")
            angles = self.position.angles(batch)
        n = x.shape[0]
        table = batch.block_tables[cache.group]
        d, dv = s.head_dim, s.value_dim
        if not s.own_kv and cache.writable:
            raise ValueError("an attention mixer without key and value projections needs the cache of another run")
        proj = rt.linear(rt.rows_of(x), self.w_qkv, slabs=True)
        norm = "none" if s.qk_norm_eps is None else ("weighted" if s.qk_norm_weight else "plain")
        coef, every = s.q_temp if s.q_temp is not None else (0.0, 0)
        # (without projections of its own only q was projected: its columns stand at the row's start all the same)
        # (with the added one the keys of a prompt portion are never cut, which the matrix-core kernel does only without a
        # window or chunk)
        wide_rows = self.pad_values and cache.v.shape[3] == d       # the values lie in rows as wide as the keys
        fast = rt.dtype == "bfloat16" and d % 16 == 0 and (d == dv or wide_rows) and not (s.sink and s.chunk is None and s.window is None) \
            and rt.ops.attention_fast_ok(s.num_heads, s.num_kv_heads, cache.page_size, table.shape[1])
        capped = fast and s.softcap is not None
        # mixed values: the source run leaves its values of this step's tokens for the runs that mix them in
        v_in = v_out = None
        if s.v_mix == "source":
            v_out = batch.step_cache["attention_v_source"] = rt.empty((n, s.v_dim), torch.float32)
        elif s.v_mix == "mix":
            v_in = batch.step_cache.get("attention_v_source")
            if v_in is None or tuple(v_in.shape) != (n, s.v_dim):
                raise ValueError("an attention mixer that mixes values in runs behind the one whose values it reads, with values of the same sizes")
        q = rt.ops.head_prepare(proj, rt.empty((n, s.q_dim), rt.act_dtype), cache.k, cache.v, batch.positions,
                                batch.seq_of_token, table, s.num_heads, s.num_kv_heads, d, dv, self.bias, norm,
                                s.qk_norm_eps or 0.0, self.q_norm, self.k_norm, coef, every,
                                write_kv=cache.writable and s.own_kv,
                                q_head_scale=self.head_temp_capped if capped else self.head_temp, v_norm_eps=s.v_norm_eps,
                                angles=angles, rotary_dim=rotary_dim, v_first_in=v_in, v_first_out=v_out, v_lambda=self.v_lambda)
        if rt.dtype == "bfloat16" and not fast:
            rt.generic_attention_launches += 1
        padded = fast and wide_rows             # results as wide as the keys, zeros beyond the value's width
        out = rt.empty((n, s.q_dim if padded else s.out_dim), rt.act_dtype)
        paged_attention(rt, batch, q, out, cache.k, cache.v, cache.page_size, table, s.num_heads, s.num_kv_heads, d, d if padded else dv,
                        self.scale, s.window, fast, owner=self, softcap=s.softcap or 0.0, chunk=s.chunk or 0, sink=s.sink)
        delta = rt.linear(out, self.w_o_padded if padded else self.w_o, slabs=True, defer=True)
        return delta if self.out_bias is None else WeightedDelta.of(rt, delta, 1.0, self.out_bias)


def paged_attention(rt, batch, q, out, k_cache, v_cache, page_size, table, n_q, n_kv, d, dv, scale, window, fast, owner=None, softcap=0.0,
                    chunk=0, sink=False):
    """The attention itself over a paged cache, for any mixer that has its queries ready: q [tokens, n_q d] -> out
    [tokens, n_q dv].  `fast`: the matrix-core kernels (prompt portions and single tokens each by their own; they
    need d == dv, or `v_cache` being `k_cache`, a value then being as wide as its key's row); else the generic kernel,
    which takes values of their own width (`v_cache` may be `k_cache` there too: a value is the first dv numbers
    of its key's row).  `softcap` c > 0: a scaled score s becomes c tanh(s / c) (with `fast`, q must come multiplied by scale / c).  `owner`: a mixer whose `_prefill_work(batch)` and `_workspace(batch)` make the work list and the
    decode workspace (else they are made here for these sizes)."""
    if fast:
        # capped scores: the builds that pass what they are given through tanh; q then comes times (scale / cap), and the cap is the scale.
        # Chunks: the builds that take the window's place for the chunk's length (work lists and splits are those of a window)
        capped = bool(softcap)
        span = chunk or window or 0
        if batch.n_portions:
            item_seq, item_tile, cuts = owner._prefill_work(batch) if owner is not None else prefill_work(rt, batch, n_q, d, span or None)
            rt.ops.attention_prefill(q, k_cache, v_cache, out, item_seq, item_tile, batch.q_start, batch.q_len, batch.positions,
                                     table, n_q, n_kv, d, softcap if capped else scale, span, cuts=cuts, capped=capped,
                                     chunked=bool(chunk), sink=sink)
        if batch.n_decode:
            rt.ops.attention_decode(q, k_cache, v_cache, out, batch.decode_rows, batch.positions, batch.seq_of_token, table,
                                    n_q, n_kv, d, softcap if capped else scale, span, batch.max_decode_ctx,
                                    owner._workspace(batch) if owner is not None else decode_workspace(rt, batch, n_q, d), capped=capped,
                                    chunked=bool(chunk), sink=sink)
    elif d == dv and v_cache is not k_cache and d <= 256 and not softcap and not chunk and not sink:
        # the float32 path, and geometries the matrix-core kernels refuse (groups above 16, odd page sizes)
        rt.ops.paged_attention_generic(q, k_cache, v_cache, out, batch.positions, batch.seq_of_token, table, n_q, n_kv, d,
                                       scale, window or 0)
    else:
        rt.ops.paged_attention_wide(q, k_cache, v_cache, out, batch.positions, batch.seq_of_token, table, n_q, n_kv, d, dv,
                                    scale, window or 0, softcap=softcap, chunk=chunk, sink=sink)
    return out


def prefill_work(rt, batch, num_heads, head_dim, window):
    """The work list of the prefill kernel: (entry, tile of 128 query rows) for every entry that brings a
    portion, the longest key range first (the kernel folds the list so that workgroups sharing a
    compute unit carry about the same load).

    A workgroup walks all keys its tile sees, one after the other.  Where the tiles times the heads are
    fewer workgroups than two a compute unit and the contexts are long (a portion of a few hundred rows
    behind thousands of keys), the keys are cut as well, at multiples of a length chosen so that the
    GPU is filled about twice: a work item is then (entry, tile, cut), and the cuts of a row are merged
    in order afterwards.  The cuts follow from the step's shape, not from a row's place in it, so a row's
    result may differ in its last bits between steps of different shapes, as between the kernels for
    portions and for single tokens.  Made by the first attention layer of a forward pass and shared by
    the others of the same geometry."""
    ops = rt.ops
    key = ("attention_prefill_work", num_heads, head_dim, window)
    work = batch.step_cache.get(key)
    if work is None:
        tile = ops.PREFILL_ROWS
        q_start = batch.host["q_start"]
        portions = [(i, n, ctx) for i, (n, ctx) in enumerate(zip(batch.host["q_len"], batch.host["ctx_len"])) if n > 1]
        tiles = [(i, t, ctx - n + min((t + 1) * tile, n) - 1, q_start[i] + t * tile, min(tile, n - t * tile))
                 for i, n, ctx in portions for t in range((n + tile - 1) // tile)]     # (entry, tile, last key, first row, rows)
        workgroups = len(tiles) * num_heads
        longest = max(last for _, _, last, _, _ in tiles) + 1
        split_keys = 0
        units = ops.compute_units(rt.device)
        if window is None and workgroups < 2 * units:
            want = -(-2 * units // workgroups)
            split_keys = max(ops.PREFILL_MIN_CUT, -(-longest // want // 64) * 64)
            if longest <= split_keys:
                split_keys = 0
        if not split_keys:
            items = sorted((-last, i, t) for i, t, last, _, _ in tiles)
            work = tuple(batch.upload([i for _, i, _ in items], [t for _, _, t in items])) + (None,)
        else:
            items, merge_rows, merge_cuts = [], [], []
            for i, t, last, row0, rows in tiles:
                cuts = last // split_keys + 1
                items.extend((-(min(last + 1, (c + 1) * split_keys) - c * split_keys), i, t, c) for c in range(cuts))
                merge_rows.extend(range(row0, row0 + rows))
                merge_cuts.extend([cuts] * rows)
            items.sort()
            most = max(merge_cuts)
            seq, til, cut, rows_d, cuts_d = batch.upload([i for _, i, _, _ in items], [t for _, _, t, _ in items],
                                                         [c for _, _, _, c in items], merge_rows, merge_cuts)
            space = ops.attention_prefill_workspace(batch.n_tokens, num_heads, head_dim, most, rt.device)
            work = (seq, til, (split_keys, cut, rows_d, cuts_d, space))
        batch.step_cache[key] = work
    return work

def decode_workspace(rt, batch, num_heads, head_dim):
    """Partial results of the split decode kernel, shared by the layers of one geometry and kept
    while the batch object lives (a recorded step keeps its own)."""
    key = ("decode_workspace", batch.n_decode, batch.max_decode_ctx, num_heads, head_dim)
    ws = batch.host.get(key)
    if ws is None:
        ws = rt.ops.attention_decode_workspace(batch.n_decode, num_heads, head_dim, batch.max_decode_ctx, rt.device)
        if not rt.merge_in_kernel:
            ws = ws[:2]         # without the counts the splits are merged by a launch of its own
        batch.host[key] = ws
    return ws


@register("mixer", "parallel_mixer")
class ParallelMixer:
    """Two mixers side by side on the same input (`ParallelMixerSpec`): delta = left_scale left(x) + right_scale right(x),
    handed on as a weighted sum of the two results, which the block adds to the residual stream term by term.  One of them
    may keep keys and values in pages and one a state of fixed size; each gets what it asked for."""

    def __init__(self, spec, runtime):
        from .base import part_class
        self.spec = spec
        self.rt = runtime
        self.sides = [part_class("mixer", side.kind)(side, runtime) for side in (spec.left, spec.right)]
        self.scales = (float(spec.left_scale), float(spec.right_scale))
        self.graph_safe = all(getattr(side, "graph_safe", False) for side in self.sides)
        if sum(side.cache_need() is not None for side in self.sides) > 1 or sum(side.state_need() is not None for side in self.sides) > 1:
            raise ValueError("of two mixers side by side at most one keeps keys and values and at most one a state")

    @staticmethod
    def _side_classes(spec):
        from .base import part_class
        return [(side, part_class("mixer", side.kind)) for side in (spec.left, spec.right)]

    @classmethod
    def params(cls, spec):
        out = {}
        for side, side_cls in cls._side_classes(spec):
            out.update({side.prefix + name: p for name, p in side_cls.params(side).items()})
        return out

    @classmethod
    def placement(cls, spec):
        out = {}
        for side, side_cls in cls._side_classes(spec):
            out.update({side.prefix + name: how for name, how in getattr(side_cls, "placement", lambda s: {})(side).items()})
        return out

    @classmethod
    def variants(cls, spec, dtype):
        out = []
        for side, side_cls in cls._side_classes(spec):
            for v in getattr(side_cls, "variants", lambda s, d: [])(side, dtype):
                if v not in out:
                    out.append(v)
        return out

    @classmethod
    def need_of(cls, spec):
        for side, side_cls in cls._side_classes(spec):
            need = getattr(side_cls, "need_of", lambda s: None)(side)
            if need is not None:
                return need
        return None

    def load(self, tensors):
        for side in self.sides:
            prefix = side.spec.prefix
            side.load({name[len(prefix):]: t for name, t in tensors.items() if name.startswith(prefix)})

    def cache_need(self):
        return next((need for need in (side.cache_need() for side in self.sides) if need is not None), None)

    def state_need(self):
        return next((need for need in (side.state_need() for side in self.sides) if need is not None), None)

    def forward(self, x, batch, cache, state):
        from ..runtime import WeightedDelta
        total = None
        for side, scale in zip(self.sides, self.scales):
            delta = side.forward(x, batch, cache if side.cache_need() is not None else None, state if side.state_need() is not None else None)
            term = WeightedDelta.of(self.rt, delta, scale)
            total = term if total is None else total.plus(term)
        return total

