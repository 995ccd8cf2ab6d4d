"""Architecture-neutral description of a decoder as data.

A model is a `ModelSpec`: sizes, a tuple of `LayerSpec`s and the order in
which they run.  Every layer names its block arrangement and gives one spec
for each part of it (mixer, feed-forward, norms); a mixer spec carries its
position-encoding spec.  A spec is a frozen dataclass whose `kind` names the
part class registered for it in `kipp_amd.parts`; all sizes and constants of
a part are fields of its spec, so no part needs to know the model it sits in.

Tensor names: a spec has a `prefix`; the part declares local parameter names
and the file name of a tensor is `prefix + local_name`.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Optional, Tuple


class ConfigError(ValueError):
    """A configuration that cannot be built: says which key and why."""


@dataclass(frozen=True)
class RMSNormSpec:
    """y = x * rsqrt(mean(x^2) + eps) * w over the last axis of `width`."""
    width: int
    eps: float
    prefix: str = ""
    kind: str = "rms_norm"
    name: str = "weight"        # the tensor's local name (file name = prefix + name)


@dataclass(frozen=True)
class OnePlusRMSNormSpec:
    """y = x * rsqrt(mean(x^2) + eps) * (1 + w): the tensor holds the weight's offset from one.  `name` is the
    tensor's local name (file name = prefix + name)."""
    width: int
    eps: float
    prefix: str = ""
    name: str = "weight"
    kind: str = "rms_norm_one_plus"


@dataclass(frozen=True)
class LayerNormSpec:
    """y = (x - mean x) / sqrt(var x + eps) * w + b over the last axis of `width`, var the mean of the squared
    deviations.  `name` and `bias_name`: the tensors' local names (file name = prefix + name)."""
    width: int
    eps: float
    prefix: str = ""
    name: str = "weight"
    bias_name: str = "bias"
    kind: str = "layer_norm"


@dataclass(frozen=True)
class RopeSpec:
    """Rotary position encoding over the first `rotary_dim` dims of a head.

    pairing "half": dim i rotates with dim i + rotary_dim/2 (the reference's
    pairing, /root/reference/src/kipp.c:2368-2382); "interleaved": dim 2i with dim 2i + 1.
    """
    head_dim: int
    theta: float
    rotary_dim: Optional[int] = None
    pairing: str = "half"
    kind: str = "rope"

    def __post_init__(self):
        rd = self.head_dim if self.rotary_dim is None else self.rotary_dim
        if rd <= 0 or rd % 2 or rd > self.head_dim:
            raise ConfigError(f"rotary_dim {rd} must be even and in (0, head_dim={self.head_dim}]")
        if not self.theta > 0:
            raise ConfigError(f"rope theta must be positive, got {self.theta}")
        if self.pairing not in ("half", "interleaved"):
            raise ConfigError(f"rope pairing {self.pairing!r} is not one of half, interleaved")


@dataclass(frozen=True)
class ScaledRopeSpec:
    """Rotary position encoding whose frequencies are stretched for contexts beyond the `original` length (the
    YaRN rule).  With f_i = theta^(-2i / rotary_dim), i < rotary_dim / 2, and
    turn(t) = rotary_dim * ln(original / (2 pi t)) / (2 ln theta), the dimension that makes t turns over the original
    length: lo = max(floor(turn(fast)), 0), hi = min(ceil(turn(slow)), rotary_dim - 1),
    ramp_i = clamp((i - lo) / max(hi - lo, 0.001), 0, 1); the frequency used is f_i / factor * ramp_i + f_i * (1 - ramp_i),
    and cosines and sines are multiplied by 0.1 ln(factor) + 1 (`magnitude`)."""
    head_dim: int
    theta: float
    factor: float
    original: float
    fast: float
    slow: float
    rotary_dim: Optional[int] = None
    pairing: str = "interleaved"
    kind: str = "rope_scaled"

    def __post_init__(self):
        rd = self.head_dim if self.rotary_dim is None else self.rotary_dim
        if rd <= 0 or rd % 2 or rd > self.head_dim:
            raise ConfigError(f"rotary_dim {rd} must be even and in (0, head_dim={self.head_dim}]")
        if not self.theta > 1:
            raise ConfigError(f"rope theta must be above 1, got {self.theta}")
        if not (self.factor > 0 and self.original > 0 and self.fast > 0 and self.slow > 0):
            raise ConfigError("rope scaling: factor, original, fast and slow must be positive")
        if self.pairing not in ("half", "interleaved"):
            raise ConfigError(f"rope pairing {self.pairing!r} is not one of half, interleaved")


@dataclass(frozen=True)
class BandScaledRopeSpec:
    """Rotary position encoding whose slow frequencies are divided by `factor`, by wavelength bands: with f_i =
    theta^(-2i / rotary_dim) and wavelength l_i = 2 pi / f_i, f_i is kept where l_i < original / high, divided by `factor`
    where l_i > original / low, and between the two blended, s = (original / l_i - low) / (high - low):
    (1 - s) f_i / factor + s f_i.  Cosines and sines keep their size."""
    head_dim: int
    theta: float
    factor: float
    low: float
    high: float
    original: float
    rotary_dim: Optional[int] = None
    pairing: str = "half"
    kind: str = "rope_band_scaled"

    def __post_init__(self):
        rd = self.head_dim if self.rotary_dim is None else self.rotary_dim
        if rd <= 0 or rd % 2 or rd > self.head_dim:
            raise ConfigError(f"rotary_dim {rd} must be even and in (0, head_dim={self.head_dim}]")
        if not self.theta > 0:
            raise ConfigError(f"rope theta must be positive, got {self.theta}")
        if not (self.factor > 0 and self.original > 0 and self.low > 0 and self.high > 0) or self.low == self.high:
            raise ConfigError("rope scaling: factor, original, low and high must be positive, low and high different")
        if self.pairing not in ("half", "interleaved"):
            raise ConfigError(f"rope pairing {self.pairing!r} is not one of half, interleaved")


@dataclass(frozen=True)
class NoPositionSpec:
    """No position encoding inside the mixer."""
    kind: str = "none"


@dataclass(frozen=True)
class AttentionSpec:
    """Causal grouped-query attention over a paged key/value cache.

    `window` None keeps every key; W keeps the last W keys (the query's own
    position included).  `qk_norm_eps` None means no per-head norm of q and k.
    `scale` None means 1/sqrt(head_dim).  `page_size` None keeps its keys in pages
    of the engine's size; P asks for pages of P tokens (a short window is served
    better by small pages), in a pool of their own.

    `bias`: q, k and v have biases (`bias_names`).  `qk_norm_weight` False: the per-head norm
    divides by the root mean square alone (no weight tensors).  `q_temp` (coef, every): the
    query at position p is multiplied by 1 + coef * ln(floor((p + 1) / every) + 1).
    `v_head_dim` D: values have D numbers a head (None: as keys).  `own_kv` False: the mixer
    has no key and value projections and reads the cache of another run (`LayerRun.cache_of`).
    `names`: local tensor names of (q, k, v, o, q norm, k norm).
    `softcap` c: a score s (scale and head factor applied) becomes c tanh(s / c) before the softmax.
    `head_temp` name: a tensor [heads] of that local name multiplies the scores of each query head.
    `v_norm_eps`: every head of a value is divided by its root mean square (no weight) before it is cached.
    `chunk` C (instead of a window): position i sees j <= i only when floor(i / C) = floor(j / C), chunks counted from
    position 0 of the sequence.  `sink`: one is added to the softmax's denominator (a key of score 0 without a value).
    `out_bias` name: the output projection has a bias of that local name.  `v_mix`: "source": this run's values (before
    any mixing) are what later runs of the same step mix in; "mix": v <- (1 - lambda) v + lambda v_source before it is
    cached, lambda the one number of the tensor `v_mix_name`, v_source the source run's values of the same token (a
    source declares the tensor too and leaves it unused).
    """
    hidden_size: int
    num_heads: int
    num_kv_heads: int
    head_dim: int
    position: object = NoPositionSpec()
    qk_norm_eps: Optional[float] = None
    window: Optional[int] = None
    scale: Optional[float] = None
    prefix: str = ""
    kind: str = "attention"
    page_size: Optional[int] = None
    bias: bool = False
    qk_norm_weight: bool = True
    q_temp: Optional[Tuple[float, int]] = None
    v_head_dim: Optional[int] = None
    own_kv: bool = True
    names: Tuple[str, ...] = ("q_proj.weight", "k_proj.weight", "v_proj.weight", "o_proj.weight", "q_norm.weight", "k_norm.weight")
    bias_names: Tuple[str, str, str] = ("q_proj.bias", "k_proj.bias", "v_proj.bias")
    softcap: Optional[float] = None
    head_temp: Optional[str] = None
    v_norm_eps: Optional[float] = None
    chunk: Optional[int] = None
    sink: bool = False
    out_bias: Optional[str] = None
    v_mix: Optional[str] = None
    v_mix_name: str = "vmix"

    def __post_init__(self):
        if self.num_heads <= 0 or self.num_kv_heads <= 0:
            raise ConfigError("attention needs at least one query head and one key/value head")
        if self.chunk is not None and (self.chunk <= 0 or self.window is not None):
            raise ConfigError("attention chunk must be positive and stands instead of a window")
        if self.v_mix not in (None, "source", "mix"):
            raise ConfigError(f"attention v_mix {self.v_mix!r} is not one of source, mix")
        if self.v_mix is not None and not self.own_kv:
            raise ConfigError("attention v_mix needs values of the mixer's own")
        if self.softcap is not None and not self.softcap > 0:
            raise ConfigError(f"attention softcap must be positive, got {self.softcap}")
        if self.v_norm_eps is not None and not self.v_norm_eps >= 0:
            raise ConfigError(f"attention v_norm_eps must not be negative, got {self.v_norm_eps}")
        if self.v_head_dim is not None and not 0 < self.v_head_dim <= 256:
            raise ConfigError(f"value head size {self.v_head_dim} unsupported: from 1 to 256")
        if self.q_temp is not None and not (len(self.q_temp) == 2 and isinstance(self.q_temp[1], int) and self.q_temp[1] > 0):
            raise ConfigError("q_temp is (coef, every) with a positive integer `every`")
        if len(self.names) != 6 or len(self.bias_names) != 3:
            raise ConfigError("names: six local tensor names; bias_names: three")
        if self.num_heads % self.num_kv_heads:
            raise ConfigError(
                f"num_attention_heads {self.num_heads} is not a multiple of "
                f"num_key_value_heads {self.num_kv_heads}")
        # any head size up to 256 runs (the float32 path and the generic kernel take it); the matrix-core attention
        # kernels of the bfloat16 path take multiples of 16 and the mixer falls back to the generic one otherwise
        if self.head_dim <= 0 or self.head_dim > 256:
            raise ConfigError(
                f"head_dim {self.head_dim} unsupported: the attention kernels take head sizes from 1 to 256")
        if self.window is not None and self.window <= 0:
            raise ConfigError(f"attention window must be positive, got {self.window}")
        if self.page_size is not None and self.page_size <= 0:
            raise ConfigError(f"attention page_size must be positive, got {self.page_size}")

    @property
    def q_dim(self) -> int:
        return self.num_heads * self.head_dim

    @property
    def kv_dim(self) -> int:
        return self.num_kv_heads * self.head_dim

    @property
    def value_dim(self) -> int:
        return self.head_dim if self.v_head_dim is None else self.v_head_dim

    @property
    def v_dim(self) -> int:
        return self.num_kv_heads * self.value_dim

    @property
    def out_dim(self) -> int:
        return self.num_heads * self.value_dim

    @property
    def plain(self) -> bool:
        """None of the extras: the mixer's first kernels (weighted norm, rotation, fused decode) apply."""
        return not self.bias and self.qk_norm_weight and self.q_temp is None and self.v_head_dim is None and self.own_kv \
            and self.softcap is None and self.head_temp is None and self.v_norm_eps is None \
            and self.chunk is None and not self.sink and self.v_mix is None


@dataclass(frozen=True)
class LatentAttentionSpec:
    """Attention whose keys and values are made from a latent of `kv_rank` numbers a token, which is all the cache keeps
    (beside `rot_dim` numbers of a rotated key part that every head shares).

    cq = N(W_dq x), q = W_uq cq, a head being [head_dim unrotated | rot_dim rotated];  W_dkv x = [c' | kr], c = N(c');
    head h: key [W_uk_h c | rot(kr)], value W_uv_h c (`v_head_dim` numbers); score = scale * q_h . key_h; position i
    sees j when 0 <= i - j < `window` (None: every j <= i); with `output_gate` head h's result is multiplied by
    sigmoid(W_g x)_h.  N is an RMS norm with a plain weight and `norm_eps`.  `position` rotates the first
    rotary_dim numbers of the rotated parts.  `names`: local tensor names of (dq, dq norm, uq, dkv, dkv norm, uk, uv, g, o)."""
    hidden_size: int
    num_heads: int
    head_dim: int
    rot_dim: int
    v_head_dim: int
    q_rank: int
    kv_rank: int
    scale: float
    norm_eps: float
    position: object = NoPositionSpec()
    window: Optional[int] = None
    output_gate: bool = True
    prefix: str = ""
    kind: str = "latent_attention"
    page_size: Optional[int] = None
    names: Tuple[str, ...] = ("dq", "dq.norm", "uq", "dkv", "dkv.norm", "uk", "uv", "g", "o")

    def __post_init__(self):
        for what, v in (("heads", self.num_heads), ("head_dim", self.head_dim), ("v_head_dim", self.v_head_dim),
                        ("q_rank", self.q_rank), ("kv_rank", self.kv_rank)):
            if v <= 0:
                raise ConfigError(f"latent attention: {what} must be positive, got {v}")
        if self.rot_dim < 0:
            raise ConfigError(f"latent attention: rot_dim must not be negative, got {self.rot_dim}")
        if self.kv_rank + self.rot_dim > 1024 or self.head_dim > 1024:
            raise ConfigError("latent attention: the cached row (kv_rank + rot_dim) and head_dim take up to 1,024 numbers")
        if self.window is not None and self.window <= 0:
            raise ConfigError(f"attention window must be positive, got {self.window}")
        if len(self.names) != 9:
            raise ConfigError("names: nine local tensor names")

    @property
    def row(self) -> int:
        """Numbers a token keeps in the cache."""
        return self.kv_rank + self.rot_dim


@dataclass(frozen=True)
class MLSTMSpec:
    """The matrix memory of xLSTM (mLSTM): per head a state S [head_dim, v_head_dim], n [head_dim] and a running maximum m
    of the gates' logarithms, all starting at zero, carried from token to token in float32.

    q = W_q x / sqrt(head_dim), k = W_k x, v = W_v x;  li = cap tanh((W_i x + b_i) / cap),
    lf = logsigmoid(cap tanh((W_f x + b_f) / cap)), cap = `gate_cap`;  m' = max(lf + m, li);
    S' = e^(lf + m - m') S + e^(li - m') k v^T, n' likewise with k;  o = S'^T q / (max(|n' . q|, e^(-m')) + 1e-6);
    every head of o over its root mean square (`norm_eps`), times the norm weight, times sigmoid(W_g x), then W_o.
    `names`: local tensor names of (q, k, v, g, o, norm, i, i bias, f, f bias)."""
    hidden_size: int
    num_heads: int
    head_dim: int
    v_head_dim: int
    gate_cap: float
    norm_eps: float
    prefix: str = ""
    kind: str = "mlstm"
    names: Tuple[str, ...] = ("q", "k", "v", "g", "o", "norm", "i", "i.b", "f", "f.b")

    def __post_init__(self):
        if self.num_heads <= 0 or self.v_head_dim <= 0 or not 0 < self.head_dim <= 1024:
            raise ConfigError("mlstm: heads and value size must be positive, key size from 1 to 1,024")
        if not self.gate_cap > 0:
            raise ConfigError(f"mlstm: gate_cap must be positive, got {self.gate_cap}")
        if len(self.names) != 10:
            raise ConfigError("names: ten local tensor names")


@dataclass(frozen=True)
class DecayAttentionSpec:
    """Linear attention with a fixed decay a head (lightning attention): per head a state S [head_dim, v_head_dim] that
    starts at zero and is carried from token to token in float32.

    q = silu(W_q x), k = silu(W_k x), v = silu(W_v x);  S_t = decay_h S_(t-1) + k_t v_t^T;  o_t = S_t^T q_t;
    all heads of o side by side over their root mean square (`norm_eps`), times the norm weight [heads v_head_dim],
    times sigmoid(W_g x), then W_o.  `decays`: one number a head.  `names`: local tensor names of (q, k, v, g, o, norm)."""
    hidden_size: int
    num_heads: int
    head_dim: int
    v_head_dim: int
    decays: Tuple[float, ...]
    norm_eps: float
    prefix: str = ""
    kind: str = "decay_attention"
    names: Tuple[str, ...] = ("q", "k", "v", "g", "o", "norm")

    def __post_init__(self):
        if self.num_heads <= 0 or self.v_head_dim <= 0 or not 0 < self.head_dim <= 1024:
            raise ConfigError("decay attention: heads and value size must be positive, key size from 1 to 1,024")
        if len(self.decays) != self.num_heads:
            raise ConfigError(f"decay attention: {len(self.decays)} decays for {self.num_heads} heads")
        if len(self.names) != 6:
            raise ConfigError("names: six local tensor names")


@dataclass(frozen=True)
class GatedDeltaSpec:
    """The gated delta rule: per head a state S [head_dim, v_head_dim] that starts at zero and is carried from token to
    token in float32, beside the last `conv_taps` - 1 inputs of the short convolutions.

    q = W_q x and k = W_k x (`num_kv_heads` heads of head_dim), v = W_v x (`num_heads` heads of v_head_dim); head h reads
    q/k head h // (num_heads / num_kv_heads).  Each channel of q, k and v passes a causal filter over its last
    `conv_taps` inputs (zeros before the start, the last tap is the current token's) and silu; every head of q and k is
    divided by sqrt(sum x^2 + `unit_eps`), q also by sqrt(head_dim).  beta = sigmoid(W_b x) and
    g = exp(-exp(A_h) softplus(W_a x + dt_h)), one a head.  S <- g S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q.
    Every head of o over its root mean square (`norm_eps`), times the norm weight [v_head_dim], times silu(W_g x), then W_o.
    `names`: local tensor names of (q, k, v, q filter, k filter, v filter, b, a, A, dt, g, o, norm)."""
    hidden_size: int
    num_heads: int
    num_kv_heads: int
    head_dim: int
    v_head_dim: int
    conv_taps: int
    norm_eps: float
    unit_eps: float = 1e-6
    prefix: str = ""
    kind: str = "gated_delta"
    names: Tuple[str, ...] = ("q", "k", "v", "q.conv", "k.conv", "v.conv", "b", "a", "A_log", "dt_bias", "g", "o", "norm")

    def __post_init__(self):
        if self.num_heads <= 0 or self.num_kv_heads <= 0 or self.num_heads % self.num_kv_heads:
            raise ConfigError(f"gated delta: heads {self.num_heads} must be a positive multiple of q/k heads {self.num_kv_heads}")
        if self.v_head_dim <= 0 or not 0 < self.head_dim <= 1024:
            raise ConfigError("gated delta: value size must be positive, key size from 1 to 1,024")
        if not 1 <= self.conv_taps <= 16:
            raise ConfigError(f"gated delta: the short convolution takes 1 to 16 taps, got {self.conv_taps}")
        if len(self.names) != 13:
            raise ConfigError("names: thirteen local tensor names")

    @property
    def channels(self) -> int:
        """Channels that pass a short convolution: q | k | v."""
        return 2 * self.num_kv_heads * self.head_dim + self.num_heads * self.v_head_dim


@dataclass(frozen=True)
class SSDSpec:
    """A selective state space layer in its dual form (Mamba-2): per head a state S [state_size, head_dim] that starts at
    zero and is carried from token to token in float32, beside the last `conv_taps` - 1 inputs of the short convolution.

    W_in x = [z | u | B | C | dt] (z, u of num_heads head_dim numbers, B, C of groups state_size, dt of num_heads); u, B and
    C pass a causal filter a channel over their last `conv_taps` inputs (with a bias; zeros before the start, the last tap
    is the current token's) and silu; dt = softplus(dt + dt_bias).  Head h reads B and C of group h // (num_heads / groups):
    S <- exp(-exp(A_h) dt) S + dt B u^T;  y = S^T C + D_h u.  y times silu(z), then an RMS norm in `norm_groups` equal
    parts (`norm_eps`) times the norm weight, then W_o.
    `names`: local tensor names of (in, conv, conv bias, dt_bias, A, D, norm, o)."""
    hidden_size: int
    num_heads: int
    head_dim: int
    state_size: int
    groups: int
    conv_taps: int
    norm_groups: int
    norm_eps: float
    prefix: str = ""
    kind: str = "ssd"
    names: Tuple[str, ...] = ("in", "conv", "conv.b", "dt_bias", "A_log", "D", "norm", "o")

    def __post_init__(self):
        if self.num_heads <= 0 or self.groups <= 0 or self.num_heads % self.groups or self.num_heads > 1024:
            raise ConfigError(f"ssd: heads {self.num_heads} must be a positive multiple of groups {self.groups}, up to 1,024")
        if self.head_dim <= 0 or not 0 < self.state_size <= 1024:
            raise ConfigError("ssd: head size must be positive, state size from 1 to 1,024")
        if not 1 <= self.conv_taps <= 16:
            raise ConfigError(f"ssd: the short convolution takes 1 to 16 taps, got {self.conv_taps}")
        if self.norm_groups <= 0 or self.inner % self.norm_groups:
            raise ConfigError(f"ssd: norm_groups {self.norm_groups} must divide heads * head size {self.inner}")
        if len(self.names) != 8:
            raise ConfigError("names: eight local tensor names")

    @property
    def inner(self) -> int:
        return self.num_heads * self.head_dim

    @property
    def channels(self) -> int:
        """Channels that pass the short convolution: u | B | C."""
        return self.inner + 2 * self.groups * self.state_size

    @property
    def in_dim(self) -> int:
        return self.inner + self.channels + self.num_heads


@dataclass(frozen=True)
class ParallelMixerSpec:
    """Two mixers side by side that read the same input: delta = left_scale * left(x) + right_scale * right(x).  At most one
    of them keeps keys and values in pages and at most one keeps state of fixed size."""
    left: object
    right: object
    left_scale: float = 1.0
    right_scale: float = 1.0
    prefix: str = ""
    kind: str = "parallel_mixer"


@dataclass(frozen=True)
class HyperConnectionSpec:
    """How one sublayer reads from and writes to `streams` copies of the residual stream: it reads sum_r in[r] X_r and
    its result y goes back as X_t <- sum_r mix[r, t] X_r + out[t] y for every t at once.  `learned` False: no tensors,
    every coefficient is one where it is on the diagonal or a vector (one copy is then the plain residual sum).
    `names`: local tensor names of (in, out, mix)."""
    streams: int
    prefix: str = ""
    learned: bool = True
    kind: str = "hyper"
    names: Tuple[str, str, str] = ("in", "out", "mix")

    def __post_init__(self):
        if not 0 < self.streams <= 8:
            raise ConfigError(f"streams must be from 1 to 8, got {self.streams}")


@dataclass(frozen=True)
class MixedHeadAttentionSpec:
    """Causal grouped-query attention without rotation whose softmax weights are mixed across heads.

    Query head h reads key/value head h // (num_heads / num_kv_heads); keys have `head_dim` values a head,
    values `v_head_dim`.  q and k are each RMS-normed over their whole projection (all heads at once, plain
    weight, `qk_norm_eps`).  score = scale * q.k - r1_h * ln(1 + r2_h * distance) (`distance_bias`).  Position i
    sees j <= i when i - j < `window` (None: every key) or j < `keep_first`.  With `sink` a learned number a head
    joins the softmax's denominator (no key, no value).  With `head_mixing` the weights of the heads are mixed
    by a [heads, heads] matrix before they meet the values of each head's own key/value head.  With
    `output_gate` the concatenated heads are multiplied by sigmoid(W_g x) before the output projection.
    `names`: the local tensor names of (q, k, v, o, q norm, k norm, r1, r2, sink, mixing matrix, gate).
    """
    hidden_size: int
    num_heads: int
    num_kv_heads: int
    head_dim: int
    v_head_dim: int
    scale: float
    qk_norm_eps: float
    window: Optional[int] = None
    keep_first: int = 0
    distance_bias: bool = True
    sink: bool = True
    head_mixing: bool = True
    output_gate: bool = True
    prefix: str = ""
    kind: str = "mixed_head_attention"
    page_size: Optional[int] = None
    names: Tuple[str, ...] = ("q", "k", "v", "o", "q.norm", "k.norm", "r1", "r2", "sink", "talk", "g")

    def __post_init__(self):
        if self.num_heads <= 0 or self.num_kv_heads <= 0 or self.num_heads % self.num_kv_heads:
            raise ConfigError(f"attention heads {self.num_heads} must be a positive multiple of key/value heads {self.num_kv_heads}")
        for what, d in (("key", self.head_dim), ("value", self.v_head_dim)):
            if d <= 0 or d > 256:
                raise ConfigError(f"{what} head size {d} unsupported: the attention kernels take head sizes from 1 to 256")
        if self.window is not None and self.window <= 0:
            raise ConfigError(f"attention window must be positive, got {self.window}")
        if self.keep_first < 0:
            raise ConfigError(f"keep_first must not be negative, got {self.keep_first}")
        if self.page_size is not None and self.page_size <= 0:
            raise ConfigError(f"attention page_size must be positive, got {self.page_size}")
        if len(self.names) != 11:
            raise ConfigError("names: eleven local tensor names")

    @property
    def q_dim(self) -> int:
        return self.num_heads * self.head_dim

    @property
    def kv_dim(self) -> int:
        return self.num_kv_heads * self.head_dim

    @property
    def v_dim(self) -> int:
        return self.num_kv_heads * self.v_head_dim

    @property
    def out_dim(self) -> int:
        return self.num_heads * self.v_head_dim


@dataclass(frozen=True)
class GatedMLPSpec:
    """down(act(gate(x)) * up(x)); `activation` is "silu" or "relu".  `names`: the local tensor names of (gate, up, down);
    `bias_names`: those of their biases (None: the projections have none)."""
    hidden_size: int
    intermediate_size: int
    activation: str = "silu"
    prefix: str = ""
    kind: str = "gated_mlp"
    names: Tuple[str, str, str] = ("gate_proj.weight", "up_proj.weight", "down_proj.weight")
    bias_names: Optional[Tuple[str, str, str]] = None

    def __post_init__(self):
        if self.intermediate_size <= 0:
            raise ConfigError("intermediate_size must be positive")
        if self.activation not in ("silu", "relu"):
            raise ConfigError(f"activation {self.activation!r} unsupported (silu, relu)")


@dataclass(frozen=True)
class RoutedMLPSpec:
    """A mixture of `experts` small feed-forwards, of which a token uses `top`: W_down_e act(W_up_e x), `activation`
    "gelu" (the exact one, with erf), "gelu_tanh", "silu", "relu" or "relu2".  p = softmax(W_router x) over all experts in float32; the
    `top` largest are chosen (the lower index first among equals) and weigh their experts' results by p / (sum of the
    chosen p + `weight_eps`).  `shared_size` I: one more expert of inner size I (tensors under `shared_prefix`) runs for
    every token and is added (None: none).  Expert e's tensors are `expert_prefix.format(e)` + (up, down).
    `activation` "relu2" is the square of relu.  `router` "sigmoid": scores s = sigmoid(W_router x); the choice goes by
    s + the tensor `correction_name` (None: no correction); with `groups` (count, keep) the experts form `count` equal groups
    of neighbours, a group's score is the sum of its two largest choice scores, and only experts of the `keep` best groups can
    be chosen; weights are s / (sum of the chosen s + `weight_eps`) * `route_scale`."""
    hidden_size: int
    experts: int
    top: int
    expert_size: int
    shared_size: Optional[int] = None
    activation: str = "gelu"
    weight_eps: float = 1e-20
    prefix: str = ""
    kind: str = "routed_mlp"
    router_name: str = "router"
    expert_prefix: str = "e{}."
    shared_prefix: str = "shared."
    names: Tuple[str, str] = ("up", "down")
    router: str = "softmax"
    correction_name: Optional[str] = None
    groups: Optional[Tuple[int, int]] = None
    route_scale: float = 1.0

    def __post_init__(self):
        if self.router not in ("softmax", "sigmoid"):
            raise ConfigError(f"routed feed-forward: router {self.router!r} is not one of softmax, sigmoid")
        if self.router == "softmax" and (self.correction_name is not None or self.groups is not None or self.route_scale != 1.0):
            raise ConfigError("routed feed-forward: a correction, groups and a scale belong to the sigmoid router")
        if self.groups is not None:
            count, keep = self.groups
            if count <= 0 or self.experts % count or not 0 < keep <= count or self.top > keep * (self.experts // count):
                raise ConfigError(f"routed feed-forward: groups {self.groups}: equal groups of the {self.experts} experts, of which "
                                  f"1 to count stay, with experts enough for the {self.top} a token uses")
        if not 0 < self.top <= self.experts:
            raise ConfigError(f"routed feed-forward: top {self.top} must be from 1 to experts {self.experts}")
        if self.experts > 1024 or self.top > 32:
            raise ConfigError("routed feed-forward: up to 1,024 experts, up to 32 a token")
        if self.expert_size <= 0 or (self.shared_size is not None and self.shared_size <= 0):
            raise ConfigError("routed feed-forward: inner sizes must be positive")
        if self.activation not in ("gelu", "gelu_tanh", "silu", "relu", "relu2"):
            raise ConfigError(f"activation {self.activation!r} unsupported (gelu, gelu_tanh, silu, relu, relu2)")


@dataclass(frozen=True)
class LayerSpec:
    """One block: `block` names the arrangement, `parts` its parts by role.

    The "pre_norm" arrangement has the roles mixer_norm, mixer, ffn_norm, ffn
    and computes x += mixer(mixer_norm(x)); x += ffn(ffn_norm(x)).  The "post_norm"
    arrangement has the same roles and norms after the sum, the sublayers reading x
    itself: x = mixer_norm(a x + mixer(x)); x = ffn_norm(a x + ffn(x)) with
    a = `residual_scale`; "post_norm_mixer" is its first half alone.  "hyper_pre_norm" keeps
    several copies of the residual stream and has the roles mixer_norm, mixer_hc, mixer,
    ffn_norm, ffn_hc, ffn (the *_hc parts say how a sublayer reads and writes the copies);
    "hyper_pre_norm_mixer" is its first half alone.  "sandwich_norm" norms a sublayer's input and its result:
    x += a mixer_post_norm(mixer(mixer_norm(x))); x += a ffn_post_norm(ffn(ffn_norm(x))), a = `residual_scale`;
    "sandwich_norm_mixer" is its first half alone.  "parallel" has the roles mixer_norm, mixer and ffn: one norm whose
    output both sublayers read, h = mixer_norm(x); x += mixer(h) + ffn(h); "parallel_mixer" is the same without a feed-forward.
    """
    parts: Tuple[Tuple[str, object], ...]
    block: str = "pre_norm"
    residual_scale: float = 1.0

    @property
    def kind(self) -> str:
        return self.block

    def part(self, role: str):
        for name, spec in self.parts:
            if name == role:
                return spec
        raise KeyError(role)


@dataclass(frozen=True)
class LayerRun:
    """One entry of the run order: run `layer`; `cache_of` names an earlier
    entry of the order (by index) whose cache this run reads instead of
    writing its own.  `add_embedding`: the embedding's output (the residual stream as it was before the first run)
    is added to the residual stream right before this run."""
    layer: int
    cache_of: Optional[int] = None
    add_embedding: bool = False


@dataclass(frozen=True)
class EmbeddingSpec:
    """x = table[token] * scale; the table is the tensor prefix + name."""
    vocab_size: int
    hidden_size: int
    prefix: str = "model.embed_tokens."
    kind: str = "embedding"
    scale: float = 1.0
    name: str = "weight"


@dataclass(frozen=True)
class HeadSpec:
    """Output head: logits = W x * scale.  `tied` aliases the embedding table; else the tensor is prefix + name."""
    vocab_size: int
    hidden_size: int
    tied: bool
    prefix: str = "lm_head."
    kind: str = "lm_head"
    scale: float = 1.0
    name: str = "weight"


@dataclass(frozen=True)
class ModelSpec:
    architecture: str
    hidden_size: int
    vocab_size: int
    max_position: int
    embedding: EmbeddingSpec
    layers: Tuple[LayerSpec, ...]
    order: Tuple[LayerRun, ...]
    final_norm: object
    head: HeadSpec
    stop_tokens: Tuple[int, ...] = field(default_factory=tuple)
    input_position: Optional[object] = None   # a position part applied to the residual stream after the embedding (None: none)
    streams: Optional[int] = None             # copies of the residual stream (None: one row a token; every layer is then no "hyper" block)
    embedding_norm: Optional[object] = None   # a norm part applied to the embedding's rows before the first layer (None: none)

    def __post_init__(self):
        hyper = [layer.block.startswith("hyper_") for layer in self.layers]
        if any(hyper) != (self.streams is not None) or (any(hyper) and not all(hyper)):
            raise ConfigError("a model keeps several copies of the residual stream in every layer or in none")
        for index, run in enumerate(self.order):
            if not 0 <= run.layer < len(self.layers):
                raise ConfigError(f"order[{index}] names layer {run.layer} of {len(self.layers)}")
            if run.cache_of is not None:
                if not 0 <= run.cache_of < index:
                    raise ConfigError(f"order[{index}] reads the cache of entry {run.cache_of}, which is not earlier")
                if self.order[run.cache_of].cache_of is not None:
                    raise ConfigError(f"order[{index}] reads the cache of an entry that has none of its own")
