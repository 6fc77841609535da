"""Specs for layer-list ("hybrid") decoders: every layer names its own token
mixer and feed-forward, so attention layers, recurrent layers and layers that
run both side by side can be ordered freely.

A spec is built from a checkpoint's ``config.json`` (see :func:`vodinex_spec`,
:func:`ruludra_spec`, :func:`vukotar_spec` and :func:`nosalorn_spec`)
or directly in code (tests, benchmarks). Nothing here fixes a size: widths,
head counts, mask sizes, filter lengths and the order of layers all come from
the config.
"""

from __future__ import annotations

from dataclasses import dataclass
from typing import Optional, Tuple, Union


@dataclass(frozen=True)
class AttnMixerSpec:
    """Softmax attention with grouped key/value heads over a local mask.

    ``chunk``: a query at position i sees keys j <= i with
    ``j // chunk == i // chunk`` (0 = no chunking). ``window``: a query sees
    at most the last ``window`` keys (0 = unlimited). Both may be combined.
    ``keep_first``: with a window, keys at positions below `keep_first` stay
    visible to every later query (at their true positions).
    ``rot_dims``: how many leading dimensions of each head are rotated
    (rotate-half pairing inside that prefix); 0 = no rotation.
    ``rot_scaling``: (factor, original length, fast turns, slow turns) of a
    YaRN frequency blend: frequencies that turn fewer than `slow` times over
    the original length are divided by `factor`, those that turn more than
    `fast` times are kept, a linear ramp over the pair index lies between,
    and cos / sin are multiplied by 0.1 ln(factor) + 1.
    ``v_mix``: the values of every such layer but the first are blended with
    the first such layer's values of the same token, v <- (1 - l) v + l v1,
    with a learned scalar l; the blend is what the cache holds."""

    heads: int
    kv_heads: int
    dim: int                 # per-head query/key size
    vdim: int                # per-head value size
    scale: float
    rot_dims: int = 0
    rot_base: float = 10000.0
    chunk: int = 0
    window: int = 0
    qk_norm: bool = True
    bias: bool = True        # q/k/v/o projections carry biases
    out_gate: bool = True    # one sigmoid gate per head on the attention output
    # a silent sink: a key of score 0 without a value takes part in the
    # normalisation, p_j = exp(s_j) / (1 + sum_j exp(s_j))
    sink: bool = False
    keep_first: int = 0
    rot_scaling: Optional[Tuple[float, float, float, float]] = None
    v_mix: bool = False
    out_bias: bool = True    # with `bias`: the output projection has one too


@dataclass(frozen=True)
class DeltaMixerSpec:
    """Gated delta rule with one decay per head and key channel, fed through
    short causal depthwise filters. ``decay_rank``/``gate_rank`` are the inner
    sizes of the two low-rank projections (read from the checkpoint)."""

    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int                # filter taps (the last tap is the current token)
    decay_rank: int = 0
    gate_rank: int = 0


@dataclass(frozen=True)
class ParallelMixerSpec:
    """An attention mixer and a delta-rule mixer reading the same input; the
    result is ``left_scale * left + right_scale * right``."""

    left: AttnMixerSpec
    right: DeltaMixerSpec
    left_scale: float
    right_scale: float


@dataclass(frozen=True)
class TiedAttnMixerSpec:
    """Windowed softmax attention whose values are its raw keys (no value
    projection): q and k are RMS-normed over the whole projection (all heads
    at once), q is scaled by 1 + temp_coef * ln(floor((p+1)/temp_every) + 1)
    at position p (temp_every 0 = off), and with `dist_bias` the score of
    query i and key j is lowered by r1[h] * ln(1 + r2[h] * (i - j)). No
    rotation. ``window``: a query sees itself and the window-1 keys before it
    (0 = unlimited)."""

    heads: int
    kv_heads: int
    dim: int
    scale: float
    window: int = 0
    temp_coef: float = 0.0
    temp_every: int = 0
    dist_bias: bool = True


@dataclass(frozen=True)
class LatentAttnMixerSpec:
    """Attention through low-rank latents, without positions: queries are
    up-projected from a normed latent of size q_rank; keys and values are
    up-projected per head from one normed latent of size kv_rank, which is all
    the cache holds. The concatenated heads pass an elementwise sigmoid gate.
    ``kv_from``: index of an earlier layer whose cached latent this layer
    reads instead of making its own."""

    heads: int
    dim: int
    vdim: int
    q_rank: int
    kv_rank: int
    scale: float
    window: int = 0
    kv_from: Optional[int] = None


@dataclass(frozen=True)
class MLSTMMixerSpec:
    """mLSTM matrix memory: per head a [dim, vdim] state with exponential
    input gate, sigmoid forget gate (both soft-capped at ``gate_cap`` in log
    space) and a running-maximum stabiliser; read-out normed per head and
    gated elementwise."""

    heads: int
    dim: int
    vdim: int
    gate_cap: float


@dataclass(frozen=True)
class DecayAttnMixerSpec:
    """Linear attention with one fixed decay per head ("lightning"
    attention): q, k, v pass silu, S_t = decay_h S_(t-1) + k_t v_t^T,
    o_t = S_t^T q_t; the concatenated heads pass one RMS norm (weighted) and
    an elementwise sigmoid gate."""

    heads: int
    dim: int
    vdim: int
    decay: Tuple[float, ...]


@dataclass(frozen=True)
class SSDMixerSpec:
    """Mamba-2 state-space layer: one projection gives gate z, input x, the
    grouped B and C and a step per head; x|B|C pass a short causal filter with
    bias and silu; per head S_t = exp(-exp(A_log) dt) S_(t-1) + dt B_t x_t^T
    ([state, vdim]), y_t = S_t^T C_t + D x_t; y * silu(z) is RMS-normed in
    `norm_groups` equal parts."""

    heads: int
    vdim: int
    state: int
    groups: int
    conv: int
    norm_groups: int = 1


MixerSpec = Union[AttnMixerSpec, DeltaMixerSpec, ParallelMixerSpec,
                  TiedAttnMixerSpec, LatentAttnMixerSpec, MLSTMMixerSpec,
                  DecayAttnMixerSpec, SSDMixerSpec]


@dataclass(frozen=True)
class RoutedExpertsSpec:
    """Mixture-of-experts feed-forward: `experts` small two-matrix
    feed-forwards of inner width `ff`, of which a token uses `top`.

    ``router``: "sigmoid" scores every expert by the sigmoid of its logit and
    weights the chosen ones by score / (sum of chosen scores + 1e-20).
    ``groups`` / ``keep``: the experts form `groups` equal runs of neighbours;
    a run is worth the sum of its `group_rank` largest scores and only experts
    of the `keep` best runs can be chosen (groups = keep = 1: no restriction).
    ``act``: "relu2" = the square of relu between the two matrices.

    ``router`` "softmax": scores are the softmax over all router outputs;
    the choice (and the worth of a group, with `group_rank` 1 its largest
    member) looks at score + `correction` (a learned vector), experts outside
    the kept groups cannot be chosen whatever their sign, and the weights are
    the plain scores times `route_scale`, not renormalised. The last
    `identity` router outputs are identity experts (result = the input) that
    have no matrices; they belong to the groups like the others.
    ``act`` "clamped_glu": three-matrix experts, g = min(gate h, limit),
    u = clamp(up h, -limit, limit), down(g sigmoid(1.702 g) (u + 1)).
    ``shared_ff``: inner width of a shared expert of the same form (own
    `shared_limit`) that every token uses, weighted by the sigmoid of a
    one-row projection of the input; 0 = none."""

    ff: int
    experts: int
    top: int
    groups: int = 1
    keep: int = 1
    group_rank: int = 2
    router: str = "sigmoid"
    act: str = "relu2"
    identity: int = 0
    route_scale: float = 1.0
    correction: bool = False
    limit: float = 0.0
    shared_ff: int = 0
    shared_limit: float = 0.0


@dataclass(frozen=True)
class HybridLayerSpec:
    kind: str                # the config's layer type
    mixer: MixerSpec
    ff: int = 0              # 0 = the layer has no (dense) feed-forward
    ff_kind: str = "dense"
    moe: Optional[RoutedExpertsSpec] = None
    # index of the layer whose parameters this layer uses (its cache is its
    # own); None = the layer has parameters of its own
    weights_of: Optional[int] = None


@dataclass(frozen=True)
class HybridSpec:
    """Engine-facing spec of a layer-list decoder (the counterpart of
    ``registry.ModelSpec`` for the uniform Qwen3 family)."""

    name: str
    arch: str
    hidden_size: int
    vocab_size: int
    layers: Tuple[HybridLayerSpec, ...]
    norm_eps: float = 1e-6
    residual_mult: float = 1.0
    max_context: int = 32768
    checkpoint_dir: Optional[str] = None
    # hashed bigram table added to the token embedding: (buckets, multiplier
    # of the previous token, multiplier of the current token); None = none
    bigram: Optional[Tuple[int, int, int]] = None
    pos_base: float = 0.0        # base of the additive sinusoid (0 = none)
    logit_scale: float = 1.0
    embed_scale: float = 1.0     # multiplies the token row
    logit_softcap: float = 0.0   # c * tanh(logits / c); 0 = none
    # behavior flags shared with ModelSpec
    reasoning: bool = False
    embedding: bool = False
    tie_embeddings: bool = False
    recommended_tp: int = 1
    num_experts: int = 0

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    def param_count(self) -> int:
        h = self.hidden_size
        n = 2 * self.vocab_size * h

        def delta(m: DeltaMixerSpec) -> int:
            qk = 2 * m.kv_heads * m.dim
            v = m.heads * m.vdim
            return (h * (qk + v + m.heads + m.decay_rank + m.gate_rank)
                    + m.decay_rank * m.heads * m.dim + m.gate_rank * v
                    + v * h + (qk + v) * m.conv)

        def attn(m: AttnMixerSpec) -> int:
            return h * (m.heads * m.dim + m.kv_heads * (m.dim + m.vdim)
                        + m.heads) + m.heads * m.vdim * h

        if self.arch == "ruludra":
            return self._sandwich_param_count()
        if self.arch == "vukotar":
            return self._parallel_param_count(active=False)
        if self.arch == "nosalorn":
            return self._prenorm_param_count(active=False)
        for layer in self.layers:
            m = layer.mixer
            if isinstance(m, ParallelMixerSpec):
                n += attn(m.left) + delta(m.right)
            elif isinstance(m, AttnMixerSpec):
                n += attn(m)
            else:
                n += delta(m)
            n += h * h                      # residual gate of the mixer
            if layer.ff:
                n += 3 * h * layer.ff + h * h
        return n

    def _sandwich_param_count(self) -> int:
        h = self.hidden_size
        n = 2 * self.vocab_size * h + h
        if self.bigram:
            n += (self.bigram[0] + 1) * h
        for i, layer in enumerate(self.layers):
            m = layer.mixer
            if isinstance(m, TiedAttnMixerSpec):
                qd, kd = m.heads * m.dim, m.kv_heads * m.dim
                n += h * (qd + kd) + qd + kd + 2 * m.heads + qd * h
            elif isinstance(m, LatentAttnMixerSpec):
                hv = m.heads * m.vdim
                n += h * m.q_rank + m.q_rank + m.heads * m.dim * m.q_rank
                if m.kv_from is None:
                    n += h * m.kv_rank + m.kv_rank
                n += (m.heads * m.dim + hv) * m.kv_rank + 2 * hv * h
            elif isinstance(m, MLSTMMixerSpec):
                hv = m.heads * m.vdim
                n += h * (2 * m.heads * m.dim + 2 * hv + 2 * m.heads)
                n += 2 * m.heads + hv + hv * h
            n += 2 * h + (i + 2)
            if layer.ff:
                n += 2 * h * layer.ff + 4 + 2 * h
        return n

    def _parallel_param_count(self, active: bool) -> int:
        """Tied embedding, Dynamic-Tanh norms, layer scales; layers that
        borrow another layer's parameters add none. `active`: count only the
        experts a token uses."""
        h = self.hidden_size
        n = self.vocab_size * h + 2 * h + 1
        for layer in self.layers:
            if layer.weights_of is not None and not active:
                continue
            m = layer.mixer
            n += 2 * h + 1 + h
            n += h * (m.heads * m.dim + m.kv_heads * (m.dim + m.vdim))
            n += m.heads * m.vdim * h
            if layer.moe:
                e = layer.moe
                n += h + e.experts * h
                n += (e.top if active else e.experts) * 2 * h * e.ff
        return n

    def _prenorm_param_count(self, active: bool) -> int:
        """Pre-norm layers with attention / decay attention / state-space
        mixers and SwiGLU or routed clamped-GLU feed-forwards."""
        h = self.hidden_size
        n = 2 * self.vocab_size * h + h
        for layer in self.layers:
            m = layer.mixer
            n += h
            if isinstance(m, AttnMixerSpec):
                cols = m.heads * m.dim + m.kv_heads * (m.dim + m.vdim)
                n += (h + 1) * cols + m.heads * m.vdim * h + int(m.v_mix)
            elif isinstance(m, DecayAttnMixerSpec):
                hv = m.heads * m.vdim
                n += h * (2 * m.heads * m.dim + 2 * hv) + hv + hv * h
            elif isinstance(m, SSDMixerSpec):
                inner, bc = m.heads * m.vdim, 2 * m.groups * m.state
                n += h * (2 * inner + bc + m.heads)
                n += (inner + bc) * (m.conv + 1) + 3 * m.heads + inner
                n += inner * h
            if layer.ff:
                n += h + 3 * h * layer.ff
            if layer.moe:
                e = layer.moe
                n += h + (e.experts + e.identity) * (h + 1)
                n += (min(e.top, e.experts) if active else e.experts) \
                    * 3 * h * e.ff
                if e.shared_ff:
                    n += 3 * h * e.shared_ff + h
        return n

    def active_param_count(self) -> int:
        if self.arch == "vukotar":
            return self._parallel_param_count(active=True)
        if self.arch == "nosalorn":
            return self._prenorm_param_count(active=True)
        return self.param_count()


def _delta_from_config(m: dict, ranks: Tuple[int, int]) -> DeltaMixerSpec:
    return DeltaMixerSpec(heads=int(m["heads"]), kv_heads=int(m["kv_heads"]),
                          dim=int(m["dim"]), vdim=int(m["vdim"]),
                          conv=int(m["conv"]), decay_rank=ranks[0],
                          gate_rank=ranks[1])


def _attn_from_config(m: dict) -> AttnMixerSpec:
    rot = m.get("rot") or {}
    mask = m.get("mask") or {}
    return AttnMixerSpec(heads=int(m["heads"]), kv_heads=int(m["kv_heads"]),
                         dim=int(m["dim"]), vdim=int(m["vdim"]),
                         scale=float(m["scale"]),
                         rot_dims=int(rot.get("dims", 0)),
                         rot_base=float(rot.get("base", 10000.0)),
                         chunk=int(mask.get("size", 0)))


def vodinex_spec(config: dict, name: str = "vodinex",
                 checkpoint_dir: Optional[str] = None,
                 tensor_shapes: Optional[dict] = None) -> HybridSpec:
    """Build the spec of a Vodinex checkpoint from its ``config.json``.

    The inner sizes of the low-rank decay and gate projections are not in the
    config; they are the row counts of ``<mixer>.a1`` / ``<mixer>.g1`` and are
    taken from ``tensor_shapes`` (tensor name -> shape). Callers that build a
    model in code pass them in the layer's mixer dict as ``decay_rank`` /
    ``gate_rank`` instead."""
    shapes = tensor_shapes or {}

    def ranks(prefix: str, m: dict) -> Tuple[int, int]:
        a = shapes.get(prefix + ".a1")
        g = shapes.get(prefix + ".g1")
        return (int(a[0]) if a else int(m.get("decay_rank", 16)),
                int(g[0]) if g else int(m.get("gate_rank", 16)))

    layers = []
    for i, lc in enumerate(config["layers"]):
        kind = lc["type"]
        m = lc["mixer"]
        if kind == "channel_delta":
            mixer: MixerSpec = _delta_from_config(m, ranks(f"l{i}.mix", m))
        elif kind == "parallel":
            mixer = ParallelMixerSpec(
                left=_attn_from_config(m["left"]),
                right=_delta_from_config(
                    m["right"], ranks(f"l{i}.mix.right", m["right"])),
                left_scale=float(m["left_scale"]),
                right_scale=float(m["right_scale"]))
        else:
            raise ValueError(f"unknown layer type {kind!r} in layer {i}")
        mlp = lc.get("mlp")
        if mlp is not None and mlp.get("kind", "dense") != "dense":
            raise ValueError(f"unknown feed-forward kind {mlp['kind']!r}")
        layers.append(HybridLayerSpec(kind=kind, mixer=mixer,
                                      ff=int(mlp["ff"]) if mlp else 0))
    return HybridSpec(name=name, arch="vodinex",
                      hidden_size=int(config["width"]),
                      vocab_size=int(config["vocab"]),
                      layers=tuple(layers),
                      norm_eps=float(config["norm"]["eps"]),
                      residual_mult=float(config["residual_mult"]),
                      max_context=int(config.get("max_context", 1 << 20)),
                      checkpoint_dir=checkpoint_dir)


def ruludra_spec(config: dict, name: str = "ruludra",
                 checkpoint_dir: Optional[str] = None,
                 tensor_shapes: Optional[dict] = None) -> HybridSpec:
    """Build the spec of a Ruludra checkpoint from its ``config.json``: a
    list of layers, each with a tied-value windowed attention, a latent
    attention or an mLSTM mixer and an optional PolyNorm feed-forward; token +
    hashed-bigram + sinusoid embedding; every layer's input is a learned
    weighted sum of the embedding output and all earlier layer results.
    A latent's query rank is `q_rank` of the mixer dict, or else the row count
    of ``<mixer>.dq`` in ``tensor_shapes``."""
    shapes = tensor_shapes or {}
    layers = []
    for i, lc in enumerate(config["layers"]):
        kind = lc["type"]
        m = lc["mixer"]
        mask = m.get("mask") or {}
        if kind == "attention":
            if int(m.get("vdim", m["dim"])) != int(m["dim"]):
                raise ValueError(f"layer {i}: values are the keys, so vdim "
                                 f"must equal dim")
            qt = m.get("q_temp") or {}
            mixer: MixerSpec = TiedAttnMixerSpec(
                heads=int(m["heads"]), kv_heads=int(m["kv_heads"]),
                dim=int(m["dim"]), scale=float(m["scale"]),
                window=int(mask.get("size", 0)),
                temp_coef=float(qt.get("coef", 0.0)),
                temp_every=int(qt.get("every", 0)))
        elif kind == "latent_attention":
            src = m.get("kv_from")
            dq = shapes.get(f"l{i}.mix.dq")
            if src is not None:
                src = int(src)
                other = config["layers"][src] if 0 <= src < i else None
                if (other is None or other["type"] != "latent_attention"
                        or other["mixer"].get("kv_from") is not None
                        or int(other["mixer"]["kv_rank"]) != int(m["kv_rank"])):
                    raise ValueError(
                        f"layer {i}: kv_from must name an earlier latent "
                        f"layer of equal kv_rank that owns its latent")
            mixer = LatentAttnMixerSpec(
                heads=int(m["heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]),
                q_rank=int(m["q_rank"]) if "q_rank" in m else int(dq[0]),
                kv_rank=int(m["kv_rank"]), scale=float(m["scale"]),
                window=int(mask.get("size", 0)), kv_from=src)
        elif kind == "mlstm":
            mixer = MLSTMMixerSpec(heads=int(m["heads"]), dim=int(m["dim"]),
                                   vdim=int(m["vdim"]),
                                   gate_cap=float(m["gate_cap"]))
        else:
            raise ValueError(f"unknown layer type {kind!r} in layer {i}")
        mlp = lc.get("mlp")
        if mlp is not None and mlp.get("kind", "dense") != "dense":
            raise ValueError(f"unknown feed-forward kind {mlp['kind']!r}")
        layers.append(HybridLayerSpec(kind=kind, mixer=mixer,
                                      ff=int(mlp["ff"]) if mlp else 0,
                                      ff_kind="poly_norm"))
    big = (config.get("embedding") or {}).get("bigram")
    return HybridSpec(
        name=name, arch="ruludra", hidden_size=int(config["width"]),
        vocab_size=int(config["vocab"]), layers=tuple(layers),
        norm_eps=float(config["norm"]["eps"]),
        max_context=int(config.get("max_context", 1 << 20)),
        checkpoint_dir=checkpoint_dir,
        bigram=(int(big["buckets"]), int(big["mul_prev"]),
                int(big["mul_cur"])) if big else None,
        pos_base=10000.0, logit_scale=float(config.get("logit_scale", 1.0)))


def vukotar_spec(config: dict, name: str = "vukotar",
                 checkpoint_dir: Optional[str] = None,
                 tensor_shapes: Optional[dict] = None) -> HybridSpec:
    """Build the spec of a Vukotar checkpoint from its ``config.json``: a
    list of parallel layers (one Dynamic-Tanh norm feeding a sink-softmax
    attention and a routed-experts feed-forward, each under a layer scale),
    layers that borrow an earlier or later layer's tensors (``weights_of``),
    scaled token embedding + sinusoid, tied and soft-capped logits."""
    raw = config["layers"]

    def owner(i: int) -> int:
        seen = set()
        while raw[i].get("weights_of") is not None:
            if i in seen:
                raise ValueError(f"layer {i}: weights_of runs in a circle")
            seen.add(i)
            i = int(raw[i]["weights_of"])
            if not 0 <= i < len(raw):
                raise ValueError("weights_of names no layer")
        return i

    layers = []
    for i, lc in enumerate(raw):
        kind = lc["type"]
        if kind != "attention":
            raise ValueError(f"unknown layer type {kind!r} in layer {i}")
        m = lc["mixer"]
        mixer = AttnMixerSpec(
            heads=int(m["heads"]), kv_heads=int(m["kv_heads"]),
            dim=int(m["dim"]), vdim=int(m["vdim"]), scale=float(m["scale"]),
            qk_norm=False, bias=False, out_gate=False, sink=True)
        mlp = lc.get("mlp")
        moe = None
        if mlp is not None:
            if mlp.get("kind") != "moe":
                raise ValueError(f"unknown feed-forward kind {mlp.get('kind')!r}")
            r = mlp["router"]
            g = r.get("groups") or {"count": 1, "keep": 1}
            moe = RoutedExpertsSpec(
                ff=int(mlp["expert"]["ff"]), experts=int(r["experts"]),
                top=int(r["top"]), groups=int(g["count"]), keep=int(g["keep"]))
            if moe.experts % moe.groups or not 1 <= moe.keep <= moe.groups:
                raise ValueError(f"layer {i}: experts must split into equal "
                                 f"groups, of which 1..groups are kept")
            if moe.top > moe.keep * (moe.experts // moe.groups):
                raise ValueError(f"layer {i}: the kept groups hold fewer "
                                 f"experts than a token uses")
        own = owner(i)
        layers.append(HybridLayerSpec(kind=kind, mixer=mixer, moe=moe,
                                      weights_of=None if own == i else own))
    for i, layer in enumerate(layers):
        if layer.weights_of is not None:
            src = layers[layer.weights_of]
            if (src.mixer, src.moe) != (layer.mixer, layer.moe):
                raise ValueError(f"layer {i} borrows the tensors of layer "
                                 f"{layer.weights_of} but differs in shape")
    return HybridSpec(
        name=name, arch="vukotar", hidden_size=int(config["width"]),
        vocab_size=int(config["vocab"]), layers=tuple(layers),
        norm_eps=float(config["norm"]["eps"]),
        max_context=int(config.get("max_context", 1 << 20)),
        checkpoint_dir=checkpoint_dir, pos_base=10000.0,
        embed_scale=float((config.get("embedding") or {}).get("scale", 1.0)),
        logit_softcap=float(config.get("logit_softcap", 0.0) or 0.0),
        tie_embeddings=True,
        num_experts=max((l.moe.experts if l.moe else 0) for l in layers))


def nosalorn_spec(config: dict, name: str = "nosalorn",
                  checkpoint_dir: Optional[str] = None,
                  tensor_shapes: Optional[dict] = None) -> HybridSpec:
    """Build the spec of a Nosalorn checkpoint from its ``config.json``: a
    list of pre-norm layers (weighted RMS norms), each with a windowed
    rotary attention (biased projections, YaRN frequencies, kept first
    tokens, values blended with the first blending layer's), a fixed-decay
    linear attention or a Mamba-2 mixer, and an optional SwiGLU or
    routed-experts feed-forward; scaled token embedding, untied head, scaled
    logits."""
    layers = []
    first_mix = None
    for i, lc in enumerate(config["layers"]):
        kind = lc["type"]
        m = lc["mixer"]
        if kind == "attention":
            rot = m.get("rot") or {}
            mask = m.get("mask") or {}
            sc = rot.get("scaling")
            mixer: MixerSpec = AttnMixerSpec(
                heads=int(m["heads"]), kv_heads=int(m["kv_heads"]),
                dim=int(m["dim"]), vdim=int(m["vdim"]),
                scale=float(m["scale"]), rot_dims=int(rot.get("dims", 0)),
                rot_base=float(rot.get("base", 10000.0)),
                window=int(mask.get("size", 0) or 0),
                keep_first=int(mask.get("keep_first", 0) or 0),
                rot_scaling=(float(sc["factor"]), float(sc["original"]),
                             float(sc["fast"]), float(sc["slow"]))
                if sc else None,
                qk_norm=False, bias=True, out_bias=False, out_gate=False,
                v_mix=bool(m.get("v_mix", False)))
            if mixer.v_mix:
                cols = mixer.kv_heads * mixer.vdim
                if first_mix is None:
                    first_mix = cols
                elif cols != first_mix:
                    raise ValueError(
                        f"layer {i}: blended values must be as wide as the "
                        f"first blending layer's ({first_mix})")
        elif kind == "lightning":
            mixer = DecayAttnMixerSpec(
                heads=int(m["heads"]), dim=int(m["dim"]), vdim=int(m["vdim"]),
                decay=tuple(float(d) for d in m["decay"]))
            if len(mixer.decay) != mixer.heads:
                raise ValueError(f"layer {i}: one decay per head is needed")
        elif kind == "mamba2":
            mixer = SSDMixerSpec(
                heads=int(m["heads"]), vdim=int(m["vdim"]),
                state=int(m["state"]), groups=int(m.get("groups", 1)),
                conv=int(m["conv"]), norm_groups=int(m.get("norm_groups", 1)))
            if mixer.heads % mixer.groups or \
                    (mixer.heads * mixer.vdim) % mixer.norm_groups:
                raise ValueError(f"layer {i}: heads must split into the "
                                 f"groups and the width into the norm groups")
        else:
            raise ValueError(f"unknown layer type {kind!r} in layer {i}")
        mlp = lc.get("mlp")
        ff, moe = 0, None
        if mlp is not None:
            fk = mlp.get("kind", "dense")
            if fk == "dense":
                ff = int(mlp["ff"])
            elif fk == "moe":
                r = mlp["router"]
                g = r.get("groups") or {"count": 1, "keep": 1}
                sh = mlp.get("shared") or {}
                moe = RoutedExpertsSpec(
                    ff=int(mlp["expert"]["ff"]), experts=int(r["experts"]),
                    top=int(r["top"]), groups=int(g["count"]),
                    keep=int(g["keep"]), group_rank=1, router="softmax",
                    act="clamped_glu", identity=int(r.get("identity", 0) or 0),
                    route_scale=float(r.get("scale", 1.0)), correction=True,
                    limit=float(mlp["expert"]["limit"]),
                    shared_ff=int(sh.get("ff", 0) or 0),
                    shared_limit=float(sh.get("limit", 0.0) or 0.0))
                n = moe.experts + moe.identity
                if n % moe.groups or not 1 <= moe.keep <= moe.groups:
                    raise ValueError(
                        f"layer {i}: experts and identity experts must split "
                        f"into equal groups, of which 1..groups are kept")
                if moe.top > moe.keep * (n // moe.groups):
                    raise ValueError(f"layer {i}: the kept groups hold fewer "
                                     f"experts than a token uses")
            else:
                raise ValueError(f"unknown feed-forward kind {fk!r}")
        layers.append(HybridLayerSpec(kind=kind, mixer=mixer, ff=ff,
                                      ff_kind="swiglu", moe=moe))
    return HybridSpec(
        name=name, arch="nosalorn", hidden_size=int(config["width"]),
        vocab_size=int(config["vocab"]), layers=tuple(layers),
        norm_eps=float(config["norm"]["eps"]),
        max_context=int(config.get("max_context", 1 << 20)),
        checkpoint_dir=checkpoint_dir,
        embed_scale=float((config.get("embedding") or {}).get("scale", 1.0)),
        logit_scale=float(config.get("logit_scale", 1.0)),
        num_experts=max([(l.moe.experts if l.moe else 0) for l in layers]
                        + [0]))
