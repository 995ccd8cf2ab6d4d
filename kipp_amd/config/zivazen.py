"""Typed configuration of the Zivazen decoder, read from its config.json.

A Zivazen model norms the embedding's rows, then runs a list of layers in which one RMS norm feeds both sublayers,
x += mixer(norm1(x)) + ff(norm1(x)), each with one of two mixers and a dense or routed feed-forward (or none):

    attention   grouped-query attention with biases, a weighted RMS norm a head on queries and keys, a rotation over part
                of the head whose slow frequencies are stretched, chunks of positions that do not see each other, one added
                to the softmax's denominator, and values mixed with those of the first such layer
    parallel    two mixers side by side on the same input, scaled and added: grouped-query attention with a rotation and a
                sliding window (`left`), and a selective state space layer in its dual form behind a short causal
                convolution, with a state of fixed size (`right`)

    dense       gate, up and down projections with biases, silu
    moe         sigmoid router with a correction of the choice, groups of experts of which the best stay, experts
                W_down relu(W_up h)^2, a shared expert

config.json names the architecture under `architecture` and gives every size and every constant that differs between
models; tensors are `embed`, `embed.norm`, `final.norm`, `head` and, for layer i, `l<i>.norm1`, `l<i>.mix.*`,
`l<i>.mlp.*`.  Keys that are not implemented are refused, never ignored.
"""
from __future__ import annotations

import copy
from dataclasses import dataclass
from typing import Optional, Tuple

from .rerizen import _float, _get, _int, _only
from .specs import (AttentionSpec, BandScaledRopeSpec, ConfigError, EmbeddingSpec, GatedMLPSpec, HeadSpec, LayerRun, LayerSpec,
                    ModelSpec, ParallelMixerSpec, RMSNormSpec, RopeSpec, RoutedMLPSpec, SSDSpec)

ARCHITECTURE = "Zivazen"
MAX_POSITION = 1 << 20      # the engine's own bound on a context (block tables are made for it); the design has none
MIXERS = ("attention", "parallel")
ATTENTION_NAMES = ("q", "k", "v", "o", "q.norm", "k.norm")


def _rotation(rot: dict, head_dim: int, where: str):
    _only(rot, ("base", "dims", "scaling"), where)
    dims, base = _int(rot, "dims", where, 2), _float(rot, "base", where)
    if rot.get("scaling") is None:
        return RopeSpec(head_dim=head_dim, theta=base, rotary_dim=dims)
    sc, at = rot["scaling"], where + "scaling."
    _only(sc, ("factor", "low", "high", "original"), at)
    return BandScaledRopeSpec(head_dim=head_dim, theta=base, factor=_float(sc, "factor", at), low=_float(sc, "low", at),
                              high=_float(sc, "high", at), original=_float(sc, "original", at), rotary_dim=dims)


def _mask_size(m: dict, where: str) -> Optional[int]:
    """The length of a chunk or window; None (every earlier position is seen) where the mixer names no mask."""
    mask = m.get("mask")
    if mask is None:
        return None
    _only(mask, ("size",), where + "mask.")
    return _int(mask, "size", where + "mask.") if mask.get("size") is not None else None


@dataclass(frozen=True)
class ZivazenConfig:
    vocab: int
    width: int
    norm_eps: float
    layers: Tuple[dict, ...]                    # as config.json gives them (checked)
    max_position: int = MAX_POSITION

    @classmethod
    def from_dict(cls, d: dict) -> "ZivazenConfig":
        _only(d, ("architecture", "architectures", "vocab", "width", "norm", "layers", "max_position", "torch_dtype"), "")
        layers = _get(d, "layers", "")
        if not isinstance(layers, list) or not layers:
            raise ConfigError("config.json layers: expected a list with at least one layer")
        norm = _get(d, "norm", "")
        _only(norm, ("eps",), "norm.")
        eps = _float(norm, "eps", "norm.")
        if not eps >= 0:
            raise ConfigError(f"config.json norm.eps: must be >= 0, got {eps}")
        cfg = cls(vocab=_int(d, "vocab", ""), width=_int(d, "width", ""), norm_eps=eps, layers=tuple(copy.deepcopy(layers)),
                  max_position=_int(d, "max_position", "") if "max_position" in d else MAX_POSITION)
        cfg.model_spec()        # checks every layer
        return cfg

    def to_dict(self) -> dict:
        d = {"architecture": ARCHITECTURE, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.norm_eps},
             "layers": copy.deepcopy(list(self.layers))}
        if self.max_position != MAX_POSITION:
            d["max_position"] = self.max_position
        return d

    # -- mixers --------------------------------------------------------------------------------
    def _attention(self, prefix: str, m: dict, where: str, v_mix: Optional[str]):
        """The design's own attention: biases, head norms, stretched rotation, chunks, the added one, mixed values."""
        _only(m, ("heads", "kv_heads", "dim", "vdim", "scale", "mask", "rot", "v_mix"), where)
        d = _int(m, "dim", where)
        return AttentionSpec(
            hidden_size=self.width, num_heads=_int(m, "heads", where), num_kv_heads=_int(m, "kv_heads", where), head_dim=d,
            position=_rotation(_get(m, "rot", where), d, where + "rot."), qk_norm_eps=self.norm_eps, scale=_float(m, "scale", where),
            prefix=prefix, bias=True, v_head_dim=_int(m, "vdim", where), names=ATTENTION_NAMES, bias_names=("q.b", "k.b", "v.b"),
            chunk=_mask_size(m, where), sink=True, out_bias="o.b", v_mix=v_mix)

    def _window_attention(self, prefix: str, m: dict, where: str):
        _only(m, ("heads", "kv_heads", "dim", "vdim", "scale", "mask", "rot"), where)
        d, dv = _int(m, "dim", where), _int(m, "vdim", where)
        return AttentionSpec(
            hidden_size=self.width, num_heads=_int(m, "heads", where), num_kv_heads=_int(m, "kv_heads", where), head_dim=d,
            position=_rotation(_get(m, "rot", where), d, where + "rot."), qk_norm_eps=None, window=_mask_size(m, where),
            scale=_float(m, "scale", where), prefix=prefix, v_head_dim=None if dv == d else dv, names=ATTENTION_NAMES)

    def _ssd(self, prefix: str, m: dict, where: str):
        _only(m, ("heads", "vdim", "state", "groups", "conv", "norm_groups"), where)
        return SSDSpec(hidden_size=self.width, num_heads=_int(m, "heads", where), head_dim=_int(m, "vdim", where),
                       state_size=_int(m, "state", where), groups=_int(m, "groups", where), conv_taps=_int(m, "conv", where),
                       norm_groups=_int(m, "norm_groups", where), norm_eps=self.norm_eps, prefix=prefix)

    def _parallel(self, i: int, m: dict, where: str):
        _only(m, ("left", "right", "left_scale", "right_scale"), where)
        return ParallelMixerSpec(left=self._window_attention(f"l{i}.mix.left.", _get(m, "left", where), where + "left."),
                                 right=self._ssd(f"l{i}.mix.right.", _get(m, "right", where), where + "right."),
                                 left_scale=_float(m, "left_scale", where), right_scale=_float(m, "right_scale", where))

    def _feed_forward(self, i: int, layer: dict):
        mlp = layer.get("mlp")
        if mlp is None:
            return None
        where = f"layers[{i}].mlp."
        kind = _get(mlp, "kind", where)
        if kind == "dense":
            _only(mlp, ("kind", "ff"), where)
            return GatedMLPSpec(self.width, _int(mlp, "ff", where), "silu", f"l{i}.mlp.", names=("gate", "up", "down"),
                                bias_names=("gate.b", "up.b", "down.b"))
        if kind == "moe":
            _only(mlp, ("kind", "expert", "router", "shared"), where)
            router = _get(mlp, "router", where)
            _only(router, ("experts", "top", "groups", "scale"), where + "router.")
            _only(_get(mlp, "expert", where), ("ff",), where + "expert.")
            groups = None
            if router.get("groups") is not None:
                _only(router["groups"], ("count", "keep"), where + "router.groups.")
                groups = (_int(router["groups"], "count", where + "router.groups."), _int(router["groups"], "keep", where + "router.groups."))
            shared = None
            if mlp.get("shared") is not None:
                _only(mlp["shared"], ("ff",), where + "shared.")
                shared = _int(mlp["shared"], "ff", where + "shared.")
            return RoutedMLPSpec(hidden_size=self.width, experts=_int(router, "experts", where + "router."),
                                 top=_int(router, "top", where + "router."), expert_size=_int(mlp["expert"], "ff", where + "expert."),
                                 shared_size=shared, activation="relu2", prefix=f"l{i}.mlp.", router="sigmoid",
                                 correction_name="correction", groups=groups,
                                 route_scale=_float(router, "scale", where + "router.") if router.get("scale") is not None else 1.0)
        raise ConfigError(f"config.json {where}kind: {kind!r} is not a feed-forward of this design (dense, moe)")

    def _norm(self, name: str) -> RMSNormSpec:
        return RMSNormSpec(self.width, self.norm_eps, name, name="")

    def model_spec(self) -> ModelSpec:
        layers = []
        source = None       # the first layer whose values the later mixing layers read
        for i, layer in enumerate(self.layers):
            if not isinstance(layer, dict):
                raise ConfigError(f"config.json layers[{i}]: expected an object")
            where = f"layers[{i}]."
            _only(layer, ("type", "mixer", "mlp"), where)
            kind = _get(layer, "type", where)
            m = _get(layer, "mixer", where)
            if not isinstance(m, dict):
                raise ConfigError(f"config.json {where}mixer: expected an object")
            if kind == "attention":
                mixes = bool(m.get("v_mix"))
                mixer = self._attention(f"l{i}.mix.", m, where + "mixer.", (("mix" if source is not None else "source") if mixes else None))
                if mixes:
                    if source is not None and (source.num_kv_heads, source.value_dim) != (mixer.num_kv_heads, mixer.value_dim):
                        raise ConfigError(f"config.json {where}mixer: values of {mixer.num_kv_heads} x {mixer.value_dim} cannot be mixed with "
                                          f"the first mixing layer's {source.num_kv_heads} x {source.value_dim}")
                    source = source or mixer
            elif kind == "parallel":
                mixer = self._parallel(i, m, where + "mixer.")
            else:
                raise ConfigError(f"config.json {where}type: {kind!r} is not a mixer of this design ({', '.join(MIXERS)})")
            parts = [("mixer_norm", self._norm(f"l{i}.norm1")), ("mixer", mixer)]
            ffn = self._feed_forward(i, layer)
            if ffn is not None:
                parts.append(("ffn", ffn))
            layers.append(LayerSpec(parts=tuple(parts), block="parallel" if ffn is not None else "parallel_mixer"))
        return ModelSpec(
            architecture=ARCHITECTURE, hidden_size=self.width, vocab_size=self.vocab, max_position=self.max_position,
            embedding=EmbeddingSpec(self.vocab, self.width, prefix="embed", name=""),
            layers=tuple(layers), order=tuple(LayerRun(i) for i in range(len(layers))), final_norm=self._norm("final.norm"),
            head=HeadSpec(self.vocab, self.width, tied=False, prefix="head", name=""),
            embedding_norm=RMSNormSpec(self.width, self.norm_eps, "embed.norm", name=""))
