"""Typed configuration of the Bebulorn decoder, read from its config.json.

A Bebulorn model is a list of layers whose sublayers are normed on both sides (a layer norm with weight and bias in
front of a sublayer and another on its result, the sum scaled by `residual_mult`), each with one of three mixers and
a dense or routed feed-forward (or none):

    lightning   linear attention with a fixed decay a head and a state of fixed size
    attention   grouped-query attention without rotation: values over their root mean square, a learned factor a
                query head, scores capped by a tanh, a sliding window
    delta       the gated delta rule behind short causal convolutions, a state of fixed size

`loop: {start, stop, times}` runs layers start .. stop-1 `times` times in a row with the same weights, every pass with
caches and states of its own; the embedding's output is added to the residual stream in front of every pass but the
first.  config.json names the architecture under `architecture` and gives every size and every constant that differs
between models; tensors are `embed`, `final.norm`, `final.norm.b`, `head` and, for layer i, `l<i>.norm1`, `l<i>.norm1b`,
`l<i>.norm2`, `l<i>.norm2b` (each with `.b`), `l<i>.mix.*`, `l<i>.mlp.*`.  Keys that are not implemented are refused,
never ignored.
"""
from __future__ import annotations

import copy
from dataclasses import dataclass
from typing import Optional, Tuple

from .rerizen import _float, _get, _int, _only
from .specs import (AttentionSpec, ConfigError, DecayAttentionSpec, EmbeddingSpec, GatedDeltaSpec, GatedMLPSpec, HeadSpec,
                    LayerNormSpec, LayerRun, LayerSpec, ModelSpec, NoPositionSpec, RoutedMLPSpec)

ARCHITECTURE = "Bebulorn"
MAX_POSITION = 1 << 20      # the engine's own bound on a context (block tables are made for it); the design has none
MIXERS = ("lightning", "attention", "delta")


@dataclass(frozen=True)
class BebulornConfig:
    vocab: int
    width: int
    norm_eps: float
    residual_mult: float
    layers: Tuple[dict, ...]                    # as config.json gives them (checked)
    loop: Optional[Tuple[int, int, int]]        # (start, stop, times)
    max_position: int = MAX_POSITION

    @classmethod
    def from_dict(cls, d: dict) -> "BebulornConfig":
        _only(d, ("architecture", "architectures", "vocab", "width", "norm", "residual_mult", "layers", "loop", "max_position", "torch_dtype"), "")
        layers = _get(d, "layers", "")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json layers: expected a list with at least one layer")
        norm = _get(d, "norm", "")
        _only(norm, ("eps",), "norm.")
        eps = _float(norm, "eps", "norm.")
        if not eps >= 0:
            raise ConfigError(f"config.json norm.eps: must be >= 0, got {eps}")
        loop = None
        if d.get("loop") is not None:
            _only(d["loop"], ("start", "stop", "times"), "loop.")
            loop = (_int(d["loop"], "start", "loop.", 0), _int(d["loop"], "stop", "loop.", 0), _int(d["loop"], "times", "loop."))
            if not loop[0] <= loop[1] <= len(layers):
                raise ConfigError(f"config.json loop: start {loop[0]} <= stop {loop[1]} <= {len(layers)} layers does not hold")
        cfg = cls(vocab=_int(d, "vocab", ""), width=_int(d, "width", ""), norm_eps=eps,
                  residual_mult=_float(d, "residual_mult", "") if d.get("residual_mult") is not None else 1.0,
                  layers=tuple(copy.deepcopy(layers)), loop=loop,
                  max_position=_int(d, "max_position", "") if "max_position" in d else MAX_POSITION)
        cfg.model_spec()        # checks every layer
        return cfg

    def to_dict(self) -> dict:
        d = {"architecture": ARCHITECTURE, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.norm_eps},
             "residual_mult": self.residual_mult, "layers": copy.deepcopy(list(self.layers))}
        if self.loop is not None:
            d["loop"] = dict(zip(("start", "stop", "times"), self.loop))
        if self.max_position != MAX_POSITION:
            d["max_position"] = self.max_position
        return d

    # -- mixers --------------------------------------------------------------------------------
    def _lightning(self, i: int, m: dict, where: str):
        _only(m, ("heads", "dim", "vdim", "decay"), where)
        heads = _int(m, "heads", where)
        decay = _get(m, "decay", where)
        if not isinstance(decay, list) or len(decay) != heads or any(isinstance(v, bool) or not isinstance(v, (int, float)) for v in decay):
            raise ConfigError(f"config.json {where}decay: expected one number for each of the {heads} heads")
        return DecayAttentionSpec(hidden_size=self.width, num_heads=heads, head_dim=_int(m, "dim", where), v_head_dim=_int(m, "vdim", where),
                                  decays=tuple(float(v) for v in decay), norm_eps=self.norm_eps, prefix=f"l{i}.mix.")

    def _attention(self, i: int, m: dict, where: str):
        _only(m, ("heads", "kv_heads", "dim", "vdim", "scale", "softcap", "mask"), where)
        window = None
        if m.get("mask") is not None:
            _only(m["mask"], ("size",), where + "mask.")
            window = _int(m["mask"], "size", where + "mask.") if m["mask"].get("size") is not None else None
        return AttentionSpec(
            hidden_size=self.width, num_heads=_int(m, "heads", where), num_kv_heads=_int(m, "kv_heads", where),
            head_dim=_int(m, "dim", where), position=NoPositionSpec(), qk_norm_eps=None, window=window, scale=_float(m, "scale", where),
            prefix=f"l{i}.mix.", v_head_dim=_int(m, "vdim", where), names=("q", "k", "v", "o", "q.norm", "k.norm"),
            softcap=_float(m, "softcap", where) if m.get("softcap") is not None else None, head_temp="temp", v_norm_eps=self.norm_eps)

    def _delta(self, i: int, m: dict, where: str):
        _only(m, ("heads", "kv_heads", "dim", "vdim", "conv"), where)
        return GatedDeltaSpec(hidden_size=self.width, num_heads=_int(m, "heads", where), num_kv_heads=_int(m, "kv_heads", where),
                              head_dim=_int(m, "dim", where), v_head_dim=_int(m, "vdim", where), conv_taps=_int(m, "conv", where),
                              norm_eps=self.norm_eps, prefix=f"l{i}.mix.")

    def _feed_forward(self, i: int, layer: dict):
        mlp = layer.get("mlp")
        if mlp is None:
            return None
        where = f"layers[{i}].mlp."
        kind = _get(mlp, "kind", where)
        if kind == "dense":
            _only(mlp, ("kind", "ff"), where)
            return GatedMLPSpec(self.width, _int(mlp, "ff", where), "relu", f"l{i}.mlp.", names=("gate", "up", "down"))
        if kind == "moe":
            _only(mlp, ("kind", "expert", "router", "shared"), where)
            router = _get(mlp, "router", where)
            _only(router, ("experts", "top"), where + "router.")
            _only(_get(mlp, "expert", where), ("ff",), where + "expert.")
            shared = None
            if mlp.get("shared") is not None:
                _only(mlp["shared"], ("ff",), where + "shared.")
                shared = _int(mlp["shared"], "ff", where + "shared.")
            return RoutedMLPSpec(hidden_size=self.width, experts=_int(router, "experts", where + "router."),
                                 top=_int(router, "top", where + "router."), expert_size=_int(mlp["expert"], "ff", where + "expert."),
                                 shared_size=shared, activation="gelu", prefix=f"l{i}.mlp.")
        raise ConfigError(f"config.json {where}kind: {kind!r} is not a feed-forward of this design (dense, moe)")

    def _norm(self, name: str) -> LayerNormSpec:
        return LayerNormSpec(self.width, self.norm_eps, name, name="", bias_name=".b")

    def model_spec(self) -> ModelSpec:
        layers = []
        for i, layer in enumerate(self.layers):
            if not isinstance(layer, dict):
                raise ConfigError(f"config.json layers[{i}]: expected an object")
            where = f"layers[{i}]."
            _only(layer, ("type", "mixer", "mlp"), where)
            kind = _get(layer, "type", where)
            m = _get(layer, "mixer", where)
            if not isinstance(m, dict):
                raise ConfigError(f"config.json {where}mixer: expected an object")
            if kind not in MIXERS:
                raise ConfigError(f"config.json {where}type: {kind!r} is not a mixer of this design ({', '.join(MIXERS)})")
            mixer = {"lightning": self._lightning, "attention": self._attention, "delta": self._delta}[kind](i, m, where + "mixer.")
            parts = [("mixer_norm", self._norm(f"l{i}.norm1")), ("mixer", mixer), ("mixer_post_norm", self._norm(f"l{i}.norm1b"))]
            ffn = self._feed_forward(i, layer)
            if ffn is not None:
                parts += [("ffn_norm", self._norm(f"l{i}.norm2")), ("ffn", ffn), ("ffn_post_norm", self._norm(f"l{i}.norm2b"))]
            layers.append(LayerSpec(parts=tuple(parts), block="sandwich_norm" if ffn is not None else "sandwich_norm_mixer",
                                    residual_scale=self.residual_mult))
        n = len(layers)
        start, stop, times = self.loop if self.loop is not None else (n, n, 1)
        order = [LayerRun(i) for i in range(start)]
        for rep in range(times):
            order += [LayerRun(i, add_embedding=rep > 0 and i == start) for i in range(start, stop)]
        order += [LayerRun(i) for i in range(stop, n)]
        return ModelSpec(
            architecture=ARCHITECTURE, hidden_size=self.width, vocab_size=self.vocab, max_position=self.max_position,
            embedding=EmbeddingSpec(self.vocab, self.width, prefix="embed", name=""),
            layers=tuple(layers), order=tuple(order), final_norm=self._norm("final.norm"),
            head=HeadSpec(self.vocab, self.width, tied=False, prefix="head", name=""))
