"""Model configurations.

Architectural dimensions of the public checkpoints named in SURVEY §2.7
(re-verified against the public HF configs at build time is impossible
offline; these are the standard published values).  Weights are random-init
unless a local HF-format directory is given (see models/weights.py).
"""
from __future__ import annotations

import json
from dataclasses import asdict, dataclass, field, replace
from pathlib import Path


@dataclass(frozen=True)
class DecoderConfig:
    name: str
    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_layers: int
    num_heads: int
    num_kv_heads: int
    head_dim: int = 128
    rms_norm_eps: float = 1e-6
    rope_theta: float = 1_000_000.0
    max_position: int = 32768
    tie_word_embeddings: bool = False
    qkv_bias: bool = True
    arch: str = "qwen2"

    def to_dict(self):
        return asdict(self)

    @property
    def norm_eps(self) -> float:
        return self.rms_norm_eps

    def param_count(self) -> int:
        H, I, L = self.hidden_size, self.intermediate_size, self.num_layers
        q = self.num_heads * self.head_dim
        kv = self.num_kv_heads * self.head_dim
        emb = self.vocab_size * H * (1 if self.tie_word_embeddings else 2)
        if self.arch == "gpt2":  # LN(w,b) x2, qkv+bias, o+bias, fc+bias, proj+bias; learned positions
            per_layer = 4 * H + H * 3 * q + 3 * q + q * H + H + 2 * H * I + I + H
            return L * per_layer + emb + self.max_position * H + 2 * H
        per_layer = H * (q + 2 * kv) + (q + 2 * kv) + q * H + 3 * H * I + 2 * H
        return L * per_layer + emb + H


@dataclass(frozen=True)
class EncoderConfig:
    name: str
    vocab_size: int = 30522
    hidden_size: int = 384
    num_layers: int = 6
    num_heads: int = 12
    intermediate_size: int = 1536
    max_position: int = 512
    type_vocab_size: int = 2
    layer_norm_eps: float = 1e-12
    pooling: str = "mean"  # "mean" | "cls"
    normalize: bool = True
    max_seq_length: int = 256  # sentence-transformers truncation
    query_prefix: str = ""

    @property
    def head_dim(self) -> int:
        return self.hidden_size // self.num_heads

    def to_dict(self):
        return asdict(self)


# ---------------------------------------------------------------------------------------------- hybrid decoders
# Decoders whose layer list is data: every layer names its sequence mixer ("parallel": softmax attention with a
# sink beside decay linear attention; "mingru": a gated recurrence) and its feed-forward, and a span of layers
# may be run several times in a row with shared weights (a loop), every pass with its own cache and state.


@dataclass(frozen=True)
class SinkAttnSpec:
    """Softmax attention with a per-head sink, GQA, partial rotary and RMS-normed values."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    rot_dims: int
    rot_base: float


@dataclass(frozen=True)
class DecayAttnSpec:
    """Linear attention with a fixed decay per head and a [dim, vdim] state per head."""
    heads: int
    dim: int
    vdim: int
    decay: tuple


@dataclass(frozen=True)
class RetentionSpec:
    """Linear attention with a fixed decay per head (no softmax, no denominator), rotary on q and k, keys scaled
    by dim^-1/2, every head's output divided by its RMS and gated by a SiLU projection."""
    heads: int
    dim: int
    vdim: int
    decay: tuple
    rot_dims: int
    rot_base: float


@dataclass(frozen=True)
class WindowAttnSpec:
    """Sliding-window attention with sigmoid weights: the values are the un-normed keys, q and k are RMS-normed per
    head, a per-head bias is added to the score, the heads are gated by a sigmoid projection."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: int


@dataclass(frozen=True)
class LatentAttnSpec:
    """Causal softmax attention over a cached latent (kv_rank) and one rotated key part (rot_dim) shared by the
    heads; queries through a latent of q_rank (0: read from the weight's shape)."""
    heads: int
    dim: int
    rot_dim: int
    vdim: int
    kv_rank: int
    q_rank: int
    scale: float
    rot_base: float
    window: int = 0  # > 0: a query sees itself and the window - 1 positions before it
    kv_from: int | None = None  # the layer whose cached latent and rotated key part this layer attends to
    q_latent: bool = True  # False: queries straight from the layer input (no query latent)
    sink: bool = False  # one learned key-less logit per head in the softmax's denominator
    gate: bool = False  # the concatenated heads are multiplied by the sigmoid of a projection of the input
    interleaved: bool = False  # rotary pairs (2i, 2i + 1) instead of (i, i + rot_dim / 2)


@dataclass(frozen=True)
class CappedAttnSpec:
    """Sliding-window softmax attention, GQA, partial rotary on halves, scores capped by softcap * tanh(s / softcap)
    (softcap 0: no cap; window 0: plain causal)."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: int
    softcap: float
    rot_dims: int
    rot_base: float


@dataclass(frozen=True)
class ChunkAttnSpec:
    """Softmax attention inside aligned blocks of ``chunk`` positions (0: plain causal), GQA, partial rotary on
    adjacent pairs, a temperature per head, a sigmoid output gate per head."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    chunk: int
    rot_dims: int
    rot_base: float


@dataclass(frozen=True)
class SSMSpec:
    """State-space mixer: ``heads`` heads of ``vdim`` channels with an [state, vdim] fp32 state each, B / C shared by
    the heads of each of ``groups`` groups, a causal convolution of ``taps`` taps in front, a gated RMS norm in
    ``norm_groups`` parts behind."""
    heads: int
    vdim: int
    state: int
    groups: int
    norm_groups: int
    taps: int

    @property
    def inner(self) -> int:
        return self.heads * self.vdim

    @property
    def conv_channels(self) -> int:
        return self.heads * self.vdim + 2 * self.groups * self.state


@dataclass(frozen=True)
class MoESpec:
    """Mixture of SiLU-gated experts: ``top`` of ``experts`` per token, chosen among the ``keep`` best of ``groups``
    equal groups of neighbours, weighted by their softmax scores; a shared expert of ``shared_ff`` (0: none) with a
    sigmoid gate per token."""
    kind: str  # "moe"
    ff: int
    experts: int
    top: int
    groups: int
    keep: int
    shared_ff: int
    limit: float | None = None  # clamped units g sigmoid(1.702 g) (u + 1), g = min(gate, limit), u = clamp(up, +-limit)
    table: bool = False  # no router: a [vocab, top] table names every token id's experts, each weighs 1 / top


@dataclass(frozen=True)
class MixerSpec:
    kind: str  # "parallel" | "mingru" | "retention" | "attention" | "latent_attention" | "mamba2"
    left: SinkAttnSpec | None = None
    right: DecayAttnSpec | None = None
    left_scale: float = 1.0
    right_scale: float = 1.0
    width: int = 0  # mingru state width
    spec: RetentionSpec | WindowAttnSpec | LatentAttnSpec | ChunkAttnSpec | CappedAttnSpec | SSMSpec | None = None  # single-mixer kinds


@dataclass(frozen=True)
class GLUSpec:
    kind: str  # "dense"
    ff: int
    limit: float | None  # clamp of the gate / up branches (None: the plain SiLU-gated unit)


@dataclass(frozen=True)
class HybridLayerSpec:
    mixer: MixerSpec
    mlp: GLUSpec | MoESpec | None


@dataclass(frozen=True)
class HybridConfig:
    name: str
    vocab_size: int
    hidden_size: int
    norm_eps: float
    layers: tuple
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 1
    arch: str = "zofesun"
    max_position: int = 1 << 20  # the design has no position limit of its own: the engine's max_model_len bounds it
    tie_word_embeddings: bool = False
    streams: int = 1  # residual streams (hyper-connections); 1 = the plain residual sum
    embed_scale: float = 1.0  # the embedding rows are multiplied by this
    residual_mult: float = 1.0  # every sublayer's output is multiplied by this before it joins the residual
    logit_softcap: float = 0.0  # > 0: logits <- cap * tanh(logits / cap)
    conv_taps: int = 0  # > 0: every mixer reads h + conv(h), a causal per-channel convolution of this many taps

    @property
    def num_layers(self) -> int:
        return len(self.layers)

    def layer_runs(self) -> list:
        """[(layer index, pass number, first of its pass)] in execution order: layers before the loop once,
        the looped span ``loop_times`` times, the rest once.  Every run has its own cache / state."""
        a, b, n = self.loop_start, self.loop_stop, len(self.layers)
        if not (0 <= a <= b <= n) or self.loop_times < 1:
            raise ValueError(f"loop [{a}, {b}) x {self.loop_times} does not fit {n} layers")
        runs = [(i, 0, False) for i in range(a)]
        for t in range(self.loop_times if b > a else 0):
            runs += [(i, t, i == a) for i in range(a, b)]
        runs += [(i, 0, False) for i in range(b, n)]
        return runs

    def to_dict(self):
        return asdict(self)

    def param_count(self) -> int:
        H = self.hidden_size
        if self.arch == "pubulix":
            n = 2 * self.vocab_size * H + 1
            for L in self.layers:
                m, a = L.mixer.kind, L.mixer.spec
                n += 1 + H * self.conv_taps + H * H + H
                if m == "attention":
                    n += H * (a.heads * a.dim + a.kv_heads * (a.dim + a.vdim)) + a.heads * a.vdim * H
                else:
                    n += H * a.heads * (a.dim + a.rot_dim) + a.kv_rank * a.heads * (a.dim + a.vdim) + a.heads
                    n += 2 * H * a.heads * a.vdim
                    if a.kv_from is None:
                        n += H * (a.kv_rank + a.rot_dim) + a.kv_rank
                if L.mlp is not None:
                    n += 1 + H * H + H + L.mlp.experts * 3 * H * L.mlp.ff + self.vocab_size * L.mlp.top
            return n
        if self.arch == "leripel":
            n = 2 * self.vocab_size * H + H + (2 * H * H if self.loop_stop > self.loop_start else 0)
            for L in self.layers:
                m, a = L.mixer.kind, L.mixer.spec
                n += H
                if m == "retention":
                    n += H * a.heads * (2 * a.dim + 2 * a.vdim) + a.heads * a.vdim * H
                elif m == "attention":
                    n += H * (a.heads * a.dim + a.kv_heads * (a.dim + a.vdim) + a.heads) + a.heads + a.heads * a.vdim * H
                else:
                    n += H * (2 * a.inner + 2 * a.groups * a.state + a.heads) + a.conv_channels * (a.taps + 1)
                    n += 3 * a.heads + a.inner + a.inner * H
                if L.mlp is not None:
                    f = L.mlp
                    n += f.experts * (3 * H * f.ff + H) + (3 * H * f.shared_ff + H if f.shared_ff else 0)
            return n
        if self.arch == "namudra":
            S = self.streams
            n = 2 * self.vocab_size * H + H
            for L in self.layers:
                m, a = L.mixer.kind, L.mixer.spec
                n += (1 if L.mlp is None else 2) * (H + (2 * S + S * S if S > 1 else 0))
                if m == "retention":
                    n += H * a.heads * (2 * a.dim + 2 * a.vdim) + a.heads * a.vdim * H
                elif m == "attention":
                    n += H * (2 * a.heads + a.kv_heads) * a.dim + 2 * a.dim + a.heads + a.heads * a.vdim * H
                else:
                    n += H * a.q_rank + a.q_rank + a.q_rank * a.heads * (a.dim + a.rot_dim)
                    n += H * (a.kv_rank + a.rot_dim) + a.kv_rank + a.kv_rank * a.heads * (a.dim + a.vdim)
                    n += a.heads * a.vdim * H
                if L.mlp is not None:
                    n += 3 * H * L.mlp.ff
            return n
        n = 2 * self.vocab_size * H + 2 * H + 1 + self.loop_times * H
        for L in self.layers:
            n += 4 * (2 * H + 1)
            m = L.mixer
            if m.kind == "mingru":
                n += 3 * m.width * H + 2 * m.width + H * m.width
            else:
                l, r = m.left, m.right
                n += H * (l.heads * l.dim + l.kv_heads * (l.dim + l.vdim)) + l.heads + l.heads * l.vdim * H
                n += H * r.heads * (2 * r.dim + 2 * r.vdim) + r.heads * r.vdim * (H + 1)
            if L.mlp is not None:
                n += 3 * H * L.mlp.ff
        return n


def hybrid_config_from_dict(d: dict, name: str = "zofesun") -> HybridConfig:
    """The design's config.json: sizes and constants are all read from it."""
    layers = []
    for e in d["layers"]:
        kind, m = e["type"], e["mixer"]
        if kind == "parallel":
            l, r = m["left"], m["right"]
            rot = l.get("rot") or {"dims": 0, "base": 1.0}  # no "rot" entry: no rotation
            left = SinkAttnSpec(int(l["heads"]), int(l.get("kv_heads", l["heads"])), int(l["dim"]), int(l["vdim"]),
                                float(l["scale"]), int(rot["dims"]), float(rot.get("base", 1.0)))
            right = DecayAttnSpec(int(r["heads"]), int(r["dim"]), int(r["vdim"]), tuple(float(x) for x in r["decay"]))
            if left.heads % left.kv_heads or left.rot_dims % 2 or left.rot_dims > left.dim:
                raise ValueError(f"bad attention sizes {l}")
            if len(right.decay) != right.heads:
                raise ValueError("one decay per linear-attention head")
            mixer = MixerSpec("parallel", left, right, float(m["left_scale"]), float(m["right_scale"]))
        elif kind == "mingru":
            mixer = MixerSpec("mingru", width=int(m["width"]))
        else:
            raise ValueError(f"unknown mixer type {kind!r}")
        f = e.get("mlp")
        if f is None:
            mlp = None
        elif f.get("kind", "dense") == "dense":
            mlp = GLUSpec("dense", int(f["ff"]), float(f["limit"]))
        else:
            raise ValueError(f"unknown feed-forward kind {f.get('kind')!r}")
        layers.append(HybridLayerSpec(mixer, mlp))
    loop = d.get("loop") or {}
    return HybridConfig(name, int(d["vocab"]), int(d["width"]), float(d["norm"]["eps"]), tuple(layers),
                        int(loop.get("start", 0)), int(loop.get("stop", 0)), int(loop.get("times", 1)))


def hybrid_config_to_dict(cfg: HybridConfig) -> dict:
    """Back to the config.json form (checkpoint export, tests)."""
    layers = []
    for L in cfg.layers:
        m = L.mixer
        if m.kind == "mingru":
            mixer = {"width": m.width}
        else:
            l, r = m.left, m.right
            mixer = {"left": {"heads": l.heads, "kv_heads": l.kv_heads, "dim": l.dim, "vdim": l.vdim, "scale": l.scale,
                              "rot": {"dims": l.rot_dims, "base": l.rot_base}},
                     "left_scale": m.left_scale,
                     "right": {"heads": r.heads, "dim": r.dim, "vdim": r.vdim, "decay": list(r.decay)},
                     "right_scale": m.right_scale}
        mlp = None if L.mlp is None else {"kind": L.mlp.kind, "ff": L.mlp.ff, "limit": L.mlp.limit}
        layers.append({"type": m.kind, "mixer": mixer, "mlp": mlp})
    return {"architecture": "Zofesun", "vocab": cfg.vocab_size, "width": cfg.hidden_size,
            "norm": {"eps": cfg.norm_eps}, "layers": layers,
            "loop": {"start": cfg.loop_start, "stop": cfg.loop_stop, "times": cfg.loop_times}}


def _glu_from_dict(f):
    if f is None:
        return None
    if f.get("kind", "dense") != "dense":
        raise ValueError(f"unknown feed-forward kind {f.get('kind')!r}")
    return GLUSpec("dense", int(f["ff"]), float(f["limit"]) if f.get("limit") is not None else None)


def namudra_config_from_dict(d: dict, name: str = "namudra") -> HybridConfig:
    """The Namudra design's config.json: a layer list of "retention" / "attention" / "latent_attention" mixers, each
    with an optional dense feed-forward; ``streams`` residual streams; an optional loop.  Every size and constant
    is read from it."""
    layers = []
    for e in d["layers"]:
        kind, m = e["type"], e["mixer"]
        if kind == "retention":
            rot = m.get("rot") or {"dims": 0, "base": 1.0}
            a = RetentionSpec(int(m["heads"]), int(m["dim"]), int(m["vdim"]), tuple(float(x) for x in m["decay"]),
                              int(rot["dims"]), float(rot.get("base", 1.0)))
            if len(a.decay) != a.heads or a.rot_dims % 2 or a.rot_dims > a.dim:
                raise ValueError(f"bad retention sizes {m}")
        elif kind == "attention":
            a = WindowAttnSpec(int(m["heads"]), int(m.get("kv_heads", m["heads"])), int(m["dim"]),
                               int(m.get("vdim", m["dim"])), float(m["scale"]), int(m["mask"]["size"]))
            if a.heads % a.kv_heads or a.vdim != a.dim or a.window < 1:
                raise ValueError(f"bad attention sizes {m} (the values are the keys: vdim == dim)")
        elif kind == "latent_attention":
            rot = m.get("rot") or {}
            a = LatentAttnSpec(int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"]), int(m["kv_rank"]),
                               int(m.get("q_rank", 0)), float(m["scale"]), float(rot.get("base", 10000.0)))
            if a.rot_dim % 2 or int(rot.get("dims", a.rot_dim)) != a.rot_dim:
                raise ValueError(f"bad latent attention sizes {m} (the rotated part is rotated whole)")
        else:
            raise ValueError(f"unknown mixer type {kind!r}")
        layers.append(HybridLayerSpec(MixerSpec(kind, spec=a), _glu_from_dict(e.get("mlp"))))
    loop = d.get("loop") or {}
    return HybridConfig(name, int(d["vocab"]), int(d["width"]), float(d["norm"]["eps"]), tuple(layers),
                        int(loop.get("start", 0)), int(loop.get("stop", 0)), int(loop.get("times", 1)),
                        arch="namudra", streams=int(d.get("streams", 1)))


def namudra_config_to_dict(cfg: HybridConfig) -> dict:
    """Back to the config.json form (checkpoint export, tests)."""
    layers = []
    for L in cfg.layers:
        a, kind = L.mixer.spec, L.mixer.kind
        if kind == "retention":
            m = {"heads": a.heads, "dim": a.dim, "vdim": a.vdim, "decay": list(a.decay),
                 "rot": {"dims": a.rot_dims, "base": a.rot_base}}
        elif kind == "attention":
            m = {"heads": a.heads, "kv_heads": a.kv_heads, "dim": a.dim, "vdim": a.vdim, "scale": a.scale,
                 "mask": {"size": a.window}}
        else:
            m = {"heads": a.heads, "dim": a.dim, "rot_dim": a.rot_dim, "vdim": a.vdim, "kv_rank": a.kv_rank,
                 "q_rank": a.q_rank, "scale": a.scale, "rot": {"dims": a.rot_dim, "base": a.rot_base}}
        mlp = None if L.mlp is None else {"kind": L.mlp.kind, "ff": L.mlp.ff}
        layers.append({"type": kind, "mixer": m, "mlp": mlp})
    return {"architecture": "Namudra", "vocab": cfg.vocab_size, "width": cfg.hidden_size, "streams": cfg.streams,
            "norm": {"eps": cfg.norm_eps}, "layers": layers,
            "loop": {"start": cfg.loop_start, "stop": cfg.loop_stop, "times": cfg.loop_times}}


def namudra_config(name: str, vocab: int, width: int, pattern: str, *, heads: int, kv_heads: int, dim: int, ff: int,
                   window: int = 1024, ret_heads: int | None = None, ret_dim: int | None = None,
                   ret_vdim: int | None = None, kv_rank: int = 256, q_rank: int = 384, rot_dim: int = 32,
                   streams: int = 2, loop=(0, 0, 1), eps: float = 1e-6, ret_ff: bool = False) -> HybridConfig:
    """A regular Namudra stack for benches and plumbing tests.  ``pattern``: one letter per layer, r = retention,
    a = windowed sigmoid attention, l = latent attention; attention layers carry a feed-forward of ``ff``."""
    rh, rdm, rvd = ret_heads or heads, ret_dim or dim, ret_vdim or dim
    decay = tuple(1.0 - 2.0 ** (-4.0 - 6.0 * i / max(1, rh - 1)) for i in range(rh))
    glu = GLUSpec("dense", ff, None)
    kinds = {
        "r": HybridLayerSpec(MixerSpec("retention", spec=RetentionSpec(rh, rdm, rvd, decay, rdm, 1e6)),
                             glu if ret_ff else None),
        "a": HybridLayerSpec(MixerSpec("attention", spec=WindowAttnSpec(heads, kv_heads, dim, dim, dim ** -0.5, window)),
                             glu),
        "l": HybridLayerSpec(MixerSpec("latent_attention", spec=LatentAttnSpec(
            heads, dim, rot_dim, dim, kv_rank, q_rank, (dim + rot_dim) ** -0.5, 1e4)), glu),
    }
    return HybridConfig(name, vocab, width, eps, tuple(kinds[c] for c in pattern), *loop, arch="namudra",
                        streams=streams)


def leripel_config_from_dict(d: dict, name: str = "leripel") -> HybridConfig:
    """The Leripel design's config.json: a layer list of "retention" / "attention" / "mamba2" mixers, each beside an
    optional mixture-of-experts feed-forward that reads the same normed input; an optional loop whose every pass
    re-enters through a projection of [x; embedding].  Every size and constant is read from it."""
    layers = []
    for e in d["layers"]:
        kind, m = e["type"], e["mixer"]
        if kind == "retention":
            a = RetentionSpec(int(m["heads"]), int(m["dim"]), int(m["vdim"]), tuple(float(x) for x in m["decay"]), 0, 1.0)
            if len(a.decay) != a.heads:
                raise ValueError(f"bad retention sizes {m}")
        elif kind == "attention":
            rot = m.get("rot") or {"dims": 0, "base": 1.0}
            mask = m.get("mask") or {"size": 0}
            a = ChunkAttnSpec(int(m["heads"]), int(m.get("kv_heads", m["heads"])), int(m["dim"]),
                              int(m.get("vdim", m["dim"])), float(m["scale"]), int(mask.get("size", 0)),
                              int(rot["dims"]), float(rot.get("base", 1.0)))
            if a.heads % a.kv_heads or a.rot_dims % 2 or a.rot_dims > a.dim or a.chunk < 0:
                raise ValueError(f"bad attention sizes {m}")
        elif kind == "mamba2":
            a = SSMSpec(int(m["heads"]), int(m["vdim"]), int(m["state"]), int(m.get("groups", 1)),
                        int(m.get("norm_groups", 1)), int(m["conv"]))
            if a.heads % a.groups or a.inner % a.norm_groups or a.taps < 1:
                raise ValueError(f"bad state-space sizes {m}")
        else:
            raise ValueError(f"unknown mixer type {kind!r}")
        f = e.get("mlp")
        if f is None:
            mlp = None
        elif f.get("kind", "moe") == "moe":
            r = f["router"]
            g = r.get("groups") or {"count": 1, "keep": 1}
            sh = f.get("shared")
            mlp = MoESpec("moe", int(f["expert"]["ff"]), int(r["experts"]), int(r["top"]), int(g["count"]),
                          int(g["keep"]), int(sh["ff"]) if sh else 0)
            if mlp.experts % mlp.groups or not 1 <= mlp.keep <= mlp.groups or not 1 <= mlp.top <= mlp.experts:
                raise ValueError(f"bad router sizes {r}")
        else:
            raise ValueError(f"unknown feed-forward kind {f.get('kind')!r}")
        layers.append(HybridLayerSpec(MixerSpec(kind, spec=a), mlp))
    loop = d.get("loop") or {}
    return HybridConfig(name, int(d["vocab"]), int(d["width"]), float(d["norm"]["eps"]), tuple(layers),
                        int(loop.get("start", 0)), int(loop.get("stop", 0)), int(loop.get("times", 1)), arch="leripel")


def leripel_config_to_dict(cfg: HybridConfig) -> dict:
    """Back to the config.json form (checkpoint export, tests)."""
    layers = []
    for L in cfg.layers:
        a, kind = L.mixer.spec, L.mixer.kind
        if kind == "retention":
            m = {"heads": a.heads, "dim": a.dim, "vdim": a.vdim, "decay": list(a.decay)}
        elif kind == "attention":
            m = {"heads": a.heads, "kv_heads": a.kv_heads, "dim": a.dim, "vdim": a.vdim, "scale": a.scale,
                 "mask": {"size": a.chunk}, "rot": {"dims": a.rot_dims, "base": a.rot_base}}
        else:
            m = {"heads": a.heads, "vdim": a.vdim, "state": a.state, "groups": a.groups,
                 "norm_groups": a.norm_groups, "conv": a.taps}
        f = L.mlp
        mlp = None if f is None else {
            "kind": "moe", "expert": {"ff": f.ff},
            "router": {"experts": f.experts, "top": f.top, "groups": {"count": f.groups, "keep": f.keep}},
            "shared": {"ff": f.shared_ff} if f.shared_ff else None}
        layers.append({"type": kind, "mixer": m, "mlp": mlp})
    return {"architecture": "Leripel", "vocab": cfg.vocab_size, "width": cfg.hidden_size,
            "norm": {"eps": cfg.norm_eps}, "layers": layers,
            "loop": {"start": cfg.loop_start, "stop": cfg.loop_stop, "times": cfg.loop_times}}


def leripel_config(name: str, vocab: int, width: int, pattern: str, *, heads: int, kv_heads: int, dim: int,
                   chunk: int = 2048, rot_dims: int | None = None, ret_heads: int | None = None,
                   ret_dim: int | None = None, ret_vdim: int | None = None, ssm_heads: int | None = None,
                   ssm_vdim: int = 64, ssm_state: int = 128, ssm_groups: int = 1, ssm_norm_groups: int = 1,
                   taps: int = 4, experts: int = 16, top: int = 4, groups=(4, 2), ff: int = 1024,
                   shared_ff: int = 0, loop=(0, 0, 1), eps: float = 1e-5, moe: bool = True) -> HybridConfig:
    """A regular Leripel stack for benches and plumbing tests.  ``pattern``: one letter per layer, r = retention,
    a = block-local attention, m = state-space mixer; every layer carries the same mixture of experts."""
    rh, rdm, rvd = ret_heads or heads, ret_dim or dim, ret_vdim or dim
    decay = tuple(1.0 - 2.0 ** (-4.0 - 6.0 * i / max(1, rh - 1)) for i in range(rh))
    sh = ssm_heads or max(1, width // ssm_vdim)
    mlp = MoESpec("moe", ff, experts, top, groups[0], groups[1], shared_ff) if moe else None
    kinds = {
        "r": MixerSpec("retention", spec=RetentionSpec(rh, rdm, rvd, decay, 0, 1.0)),
        "a": MixerSpec("attention", spec=ChunkAttnSpec(heads, kv_heads, dim, dim, dim ** -0.5, chunk,
                                                       dim // 2 if rot_dims is None else rot_dims, 1e4)),
        "m": MixerSpec("mamba2", spec=SSMSpec(sh, ssm_vdim, ssm_state, ssm_groups, ssm_norm_groups, taps)),
    }
    return HybridConfig(name, vocab, width, eps, tuple(HybridLayerSpec(kinds[c], mlp) for c in pattern), *loop,
                        arch="leripel")


def pubulix_config_from_dict(d: dict, name: str = "pubulix") -> HybridConfig:
    """The Pubulix design's config.json: a layer list of "attention" (capped sliding-window GQA) and
    "latent_attention" (sliding-window attention over a cached latent, with a sink and an output gate; a layer may
    attend to an earlier layer's cache) mixers, each with an optional table-routed mixture of clamped experts; a
    scalar-weight RMS norm, an input convolution in front of every mixer, sigmoid-gated residual branches.  Every
    size and constant is read from it."""
    layers = []
    for i, e in enumerate(d["layers"]):
        kind, m = e["type"], e["mixer"]
        rot = m.get("rot") or {"dims": 0, "base": 1.0}
        mask = m.get("mask") or {"size": 0}
        if kind == "attention":
            a = CappedAttnSpec(int(m["heads"]), int(m.get("kv_heads", m["heads"])), int(m["dim"]),
                               int(m.get("vdim", m["dim"])), float(m["scale"]), int(mask.get("size", 0)),
                               float(m.get("softcap") or 0.0), int(rot["dims"]), float(rot.get("base", 1.0)))
            if a.heads % a.kv_heads or a.rot_dims % 2 or a.rot_dims > a.dim or a.window < 0 or a.softcap < 0:
                raise ValueError(f"bad attention sizes {m}")
        elif kind == "latent_attention":
            src = m.get("kv_from")
            a = LatentAttnSpec(int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"]), int(m["kv_rank"]), 0,
                               float(m["scale"]), float(rot.get("base", 10000.0)), int(mask.get("size", 0)),
                               None if src is None else int(src), q_latent=False, sink=True, gate=True,
                               interleaved=True)
            if a.rot_dim % 2 or int(rot.get("dims", a.rot_dim)) != a.rot_dim or a.window < 0:
                raise ValueError(f"bad latent attention sizes {m} (the rotated part is rotated whole)")
            if a.kv_from is not None:
                o = layers[a.kv_from].mixer if 0 <= a.kv_from < i else None
                if (o is None or o.kind != "latent_attention" or o.spec.kv_from is not None
                        or (o.spec.kv_rank, o.spec.rot_dim, o.spec.rot_base) != (a.kv_rank, a.rot_dim, a.rot_base)):
                    raise ValueError(f"layer {i}: kv_from {a.kv_from} names no earlier latent layer with a cache of "
                                     "its own and the same latent size and rotation")
        else:
            raise ValueError(f"unknown mixer type {kind!r}")
        f = e.get("mlp")
        if f is None:
            mlp = None
        elif f.get("kind", "moe") == "moe":
            r = f["router"]
            lim = f["expert"].get("limit")
            mlp = MoESpec("moe", int(f["expert"]["ff"]), int(r["experts"]), int(r["top"]), 1, 1, 0,
                          None if lim is None else float(lim), table=True)
            if not 1 <= mlp.top <= mlp.experts:
                raise ValueError(f"bad expert table sizes {r}")
        else:
            raise ValueError(f"unknown feed-forward kind {f.get('kind')!r}")
        layers.append(HybridLayerSpec(MixerSpec(kind, spec=a), mlp))
    taps = int((d.get("canon") or {}).get("taps", 0))
    if taps < 0:
        raise ValueError("canon.taps < 0")
    return HybridConfig(name, int(d["vocab"]), int(d["width"]), float(d["norm"]["eps"]), tuple(layers), arch="pubulix",
                        embed_scale=float((d.get("embedding") or {}).get("scale", 1.0)),
                        residual_mult=float(d.get("residual_mult", 1.0)),
                        logit_softcap=float(d.get("logit_softcap") or 0.0), conv_taps=taps)


def pubulix_config_to_dict(cfg: HybridConfig) -> dict:
    """Back to the config.json form (checkpoint export, tests)."""
    layers = []
    for L in cfg.layers:
        a, kind = L.mixer.spec, L.mixer.kind
        if kind == "attention":
            m = {"heads": a.heads, "kv_heads": a.kv_heads, "dim": a.dim, "vdim": a.vdim, "scale": a.scale,
                 "softcap": a.softcap, "mask": {"size": a.window}, "rot": {"dims": a.rot_dims, "base": a.rot_base}}
        else:
            m = {"heads": a.heads, "dim": a.dim, "rot_dim": a.rot_dim, "vdim": a.vdim, "kv_rank": a.kv_rank,
                 "scale": a.scale, "mask": {"size": a.window}, "rot": {"dims": a.rot_dim, "base": a.rot_base}}
            if a.kv_from is not None:
                m["kv_from"] = a.kv_from
        f = L.mlp
        mlp = None if f is None else {"kind": "moe", "expert": {"ff": f.ff, "limit": f.limit},
                                      "router": {"experts": f.experts, "top": f.top}}
        layers.append({"type": kind, "mixer": m, "mlp": mlp})
    return {"architecture": "Pubulix", "vocab": cfg.vocab_size, "width": cfg.hidden_size,
            "norm": {"eps": cfg.norm_eps}, "canon": {"taps": cfg.conv_taps}, "embedding": {"scale": cfg.embed_scale},
            "residual_mult": cfg.residual_mult, "logit_softcap": cfg.logit_softcap, "layers": layers}


def pubulix_config(name: str, vocab: int, width: int, pattern: str, *, heads: int, kv_heads: int, dim: int,
                   window: int = 1024, softcap: float = 50.0, rot_dims: int | None = None, lat_heads: int | None = None,
                   lat_dim: int | None = None, lat_vdim: int | None = None, kv_rank: int = 256, rot_dim: int = 32,
                   lat_window: int = 2048, experts: int = 16, top: int = 2, ff: int = 1024, limit: float = 7.0,
                   taps: int = 4, eps: float = 1e-5, embed_scale: float = 1.0, residual_mult: float = 1.0,
                   logit_softcap: float = 30.0, moe: bool = True) -> HybridConfig:
    """A regular Pubulix stack for benches and plumbing tests.  ``pattern``: one letter per layer, a = capped
    sliding-window attention, l = latent attention with a cache of its own, s = latent attention over the cache of
    the nearest "l" before it; every layer carries the same table-routed experts."""
    lh, ld, lv = lat_heads or heads, lat_dim or dim, lat_vdim or dim
    mlp = MoESpec("moe", ff, experts, top, 1, 1, 0, limit, table=True) if moe else None
    layers, last = [], None
    for i, c in enumerate(pattern):
        if c == "a":
            spec = CappedAttnSpec(heads, kv_heads, dim, dim, dim ** -0.5, window, softcap,
                                  dim if rot_dims is None else rot_dims, 1e4)
            layers.append(HybridLayerSpec(MixerSpec("attention", spec=spec), mlp))
            continue
        if c == "l":
            last = i
        elif last is None:
            raise ValueError("an 's' layer needs an 'l' layer before it")
        spec = LatentAttnSpec(lh, ld, rot_dim, lv, kv_rank, 0, (ld + rot_dim) ** -0.5, 1e4, lat_window,
                              last if c == "s" else None, q_latent=False, sink=True, gate=True, interleaved=True)
        layers.append(HybridLayerSpec(MixerSpec("latent_attention", spec=spec), mlp))
    return HybridConfig(name, vocab, width, eps, tuple(layers), arch="pubulix", embed_scale=embed_scale,
                        residual_mult=residual_mult, logit_softcap=logit_softcap, conv_taps=taps)


def zofesun_config(name: str, vocab: int, width: int, n_layers: int, *, heads: int, kv_heads: int, dim: int,
                   vdim: int, lin_heads: int, lin_dim: int, lin_vdim: int, ff: int, mingru_every: int = 0,
                   rot_dims: int | None = None, rot_base: float = 10000.0, loop=(0, 0, 1), limit: float = 7.0,
                   eps: float = 1e-5) -> HybridConfig:
    """A regular Zofesun stack for benches and plumbing tests: ``n_layers`` parallel layers, every
    ``mingru_every``-th one (if any) a minGRU layer instead, decays spread over the linear heads."""
    left = SinkAttnSpec(heads, kv_heads, dim, vdim, dim ** -0.5, dim if rot_dims is None else rot_dims, rot_base)
    decay = tuple(1.0 - 2.0 ** (-2.0 - 6.0 * i / max(1, lin_heads - 1)) for i in range(lin_heads))
    right = DecayAttnSpec(lin_heads, lin_dim, lin_vdim, decay)
    par = HybridLayerSpec(MixerSpec("parallel", left, right, 0.7, 0.9), GLUSpec("dense", ff, limit))
    gru = HybridLayerSpec(MixerSpec("mingru", width=width), GLUSpec("dense", ff, limit))
    layers = tuple(gru if mingru_every and (i + 1) % mingru_every == 0 else par for i in range(n_layers))
    return HybridConfig(name, vocab, width, eps, layers, *loop)


HYBRIDS = {
    # plumbing-test sizes (CPU tier) and two bench sizes shaped like the layers of a 1.5B / 7B decoder
    "zofesun-tiny": zofesun_config("zofesun-tiny", 384, 128, 3, heads=4, kv_heads=2, dim=48, vdim=16, lin_heads=2,
                                   lin_dim=16, lin_vdim=24, ff=192, mingru_every=2, rot_dims=16, loop=(1, 3, 2)),
    "zofesun-1b": zofesun_config("zofesun-1b", 32768, 1536, 8, heads=12, kv_heads=2, dim=128, vdim=128,
                                 lin_heads=12, lin_dim=128, lin_vdim=128, ff=8960, mingru_every=4),
    "zofesun-7b": zofesun_config("zofesun-7b", 32768, 3584, 4, heads=28, kv_heads=4, dim=128, vdim=128,
                                 lin_heads=28, lin_dim=128, lin_vdim=128, ff=18944, mingru_every=4),
    # Namudra: a plumbing-test size and two bench sizes with the layer shapes of a 1.5B / 7B decoder
    "namudra-tiny": namudra_config("namudra-tiny", 320, 96, "ralr", heads=4, kv_heads=2, dim=16, ff=160, window=9,
                                   ret_heads=3, ret_dim=8, ret_vdim=24, kv_rank=32, q_rank=24, rot_dim=8, streams=2,
                                   loop=(1, 3, 2)),
    "namudra-1b": namudra_config("namudra-1b", 32768, 1536, "ralarala", heads=12, kv_heads=2, dim=128, ff=8960,
                                 window=1024, kv_rank=192, q_rank=384, rot_dim=64, ret_ff=True),
    "namudra-7b": namudra_config("namudra-7b", 32768, 3584, "rala", heads=28, kv_heads=4, dim=128, ff=18944,
                                 window=1024, kv_rank=192, q_rank=768, rot_dim=64, ret_ff=True),
    # Leripel: a plumbing-test size and two bench sizes with the layer shapes of a 1.5B / 7B decoder (the routed
    # experts' active width top * ff plus the shared expert equals the dense decoders' feed-forward width)
    "leripel-tiny": leripel_config("leripel-tiny", 320, 96, "rama", heads=4, kv_heads=2, dim=16, chunk=9, rot_dims=8,
                                   ret_heads=3, ret_dim=8, ret_vdim=24, ssm_heads=6, ssm_vdim=8, ssm_state=12,
                                   ssm_groups=2, ssm_norm_groups=3, experts=6, top=2, groups=(3, 2), ff=40,
                                   shared_ff=56, loop=(1, 3, 2)),
    "leripel-1b": leripel_config("leripel-1b", 32768, 1536, "ramarama", heads=12, kv_heads=2, dim=128, chunk=1024,
                                 ssm_vdim=64, ssm_state=128, experts=16, top=4, groups=(4, 2), ff=1792,
                                 shared_ff=1792),
    "leripel-7b": leripel_config("leripel-7b", 32768, 3584, "rama", heads=28, kv_heads=4, dim=128, chunk=1024,
                                 ssm_vdim=64, ssm_state=128, experts=16, top=4, groups=(4, 2), ff=3840,
                                 shared_ff=3584),
    # Pubulix: a plumbing-test size and two bench sizes with the layer shapes of a 1.5B / 7B decoder (the experts'
    # active width top * ff equals the dense decoders' feed-forward width)
    "pubulix-tiny": pubulix_config("pubulix-tiny", 320, 96, "alas", heads=4, kv_heads=2, dim=16, window=9, softcap=8.0,
                                   rot_dims=8, lat_heads=3, lat_dim=8, lat_vdim=12, kv_rank=24, rot_dim=8,
                                   lat_window=13, experts=6, top=2, ff=40, limit=1.5, taps=3, embed_scale=2.0,
                                   residual_mult=0.5),
    "pubulix-1b": pubulix_config("pubulix-1b", 32768, 1536, "alasalas", heads=12, kv_heads=2, dim=128, window=1024,
                                 lat_heads=12, kv_rank=192, rot_dim=64, lat_window=2048, experts=16, top=4, ff=2240),
    "pubulix-7b": pubulix_config("pubulix-7b", 32768, 3584, "alas", heads=28, kv_heads=4, dim=128, window=1024,
                                 lat_heads=28, kv_rank=192, rot_dim=64, lat_window=2048, experts=16, top=4, ff=4736),
}


def config_from_dir(path) -> DecoderConfig | HybridConfig:
    """The decoder config a checkpoint directory's config.json describes: the hybrid design by its
    ``architecture`` key, the HF families by ``model_type``."""
    d = json.loads((Path(path) / "config.json").read_text())
    arch = str(d.get("architecture", "")).lower()
    if arch == "zofesun":
        return hybrid_config_from_dict(d, Path(path).name or "zofesun")
    if arch == "namudra":
        return namudra_config_from_dict(d, Path(path).name or "namudra")
    if arch == "leripel":
        return leripel_config_from_dict(d, Path(path).name or "leripel")
    if arch == "pubulix":
        return pubulix_config_from_dict(d, Path(path).name or "pubulix")
    mt = str(d.get("model_type", "")).lower()
    if mt == "gpt2":
        return DecoderConfig(Path(path).name, d["vocab_size"], d["n_embd"], d.get("n_inner") or 4 * d["n_embd"],
                             d["n_layer"], d["n_head"], d["n_head"], d["n_embd"] // d["n_head"],
                             d.get("layer_norm_epsilon", 1e-5), 0.0, d.get("n_positions", 1024), True, True, "gpt2")
    if mt.startswith("qwen2"):
        hd = d.get("head_dim") or d["hidden_size"] // d["num_attention_heads"]
        return DecoderConfig(Path(path).name, d["vocab_size"], d["hidden_size"], d["intermediate_size"],
                             d["num_hidden_layers"], d["num_attention_heads"],
                             d.get("num_key_value_heads", d["num_attention_heads"]), hd, d.get("rms_norm_eps", 1e-6),
                             d.get("rope_theta", 1e6), d.get("max_position_embeddings", 32768),
                             d.get("tie_word_embeddings", False))
    raise ValueError(f"config.json of {path} names no architecture this engine serves")


DECODERS = {
    # reference deployment (helm/values.yaml:67) — served unquantised here
    "qwen2.5-coder-7b": DecoderConfig("qwen2.5-coder-7b", 152064, 3584, 18944, 28, 28, 4),
    # code default (rag_shared/config.py:29)
    "qwen2.5-3b": DecoderConfig("qwen2.5-3b", 151936, 2048, 11008, 36, 16, 2, tie_word_embeddings=True),
    "qwen2-0.5b": DecoderConfig("qwen2-0.5b", 151936, 896, 4864, 24, 14, 2, 64, tie_word_embeddings=True),
    "qwen2-1.5b": DecoderConfig("qwen2-1.5b", 151936, 1536, 8960, 28, 12, 2, tie_word_embeddings=True),
    "qwen2-7b": DecoderConfig("qwen2-7b", 152064, 3584, 18944, 28, 28, 4),
    "qwen2-72b": DecoderConfig("qwen2-72b", 152064, 8192, 29568, 80, 64, 8),
    # tiny configs for tests / CPU plumbing
    "qwen2-tiny": DecoderConfig("qwen2-tiny", 512, 256, 512, 2, 4, 2, 64, max_position=4096),
    "qwen2-small": DecoderConfig("qwen2-small", 4096, 512, 1408, 4, 8, 2, 64, max_position=8192),
    # Qwen2-72B's head layout scaled down (GQA 8:1 -> 16 q / 8 kv heads): TP = 8 leaves each rank 2 q heads and
    # one kv head, as the 72B's 8 / 1 at TP = 8 (BASELINE config 4's command form, rehearsed on the host)
    "qwen2-tiny-tp8": DecoderConfig("qwen2-tiny-tp8", 512, 512, 1024, 2, 16, 8, 32, max_position=4096),
    # GPT-2 family (BASELINE config 1: "GPT-2-small greedy answer"): pre-LN,
    # learned absolute positions, GELU(tanh) MLP, MHA, tied LM head
    "gpt2": DecoderConfig("gpt2", 50257, 768, 3072, 12, 12, 12, 64, 1e-5, 0.0, 1024, True, True, "gpt2"),
    "gpt2-medium": DecoderConfig("gpt2-medium", 50257, 1024, 4096, 24, 16, 16, 64, 1e-5, 0.0, 1024, True, True,
                                 "gpt2"),
    "gpt2-large": DecoderConfig("gpt2-large", 50257, 1280, 5120, 36, 20, 20, 64, 1e-5, 0.0, 1024, True, True,
                                "gpt2"),
    "gpt2-xl": DecoderConfig("gpt2-xl", 50257, 1600, 6400, 48, 25, 25, 64, 1e-5, 0.0, 1024, True, True, "gpt2"),
    "gpt2-tiny": DecoderConfig("gpt2-tiny", 512, 256, 1024, 2, 4, 4, 64, 1e-5, 0.0, 512, True, True, "gpt2"),
}

ENCODERS = {
    # reference default (rag_shared/config.py:24)
    "all-minilm-l6-v2": EncoderConfig("all-minilm-l6-v2", hidden_size=384, num_layers=6, num_heads=12,
                                      intermediate_size=1536, pooling="mean", max_seq_length=256),
    # README claim (README.md:139)
    "e5-small-v2": EncoderConfig("e5-small-v2", hidden_size=384, num_layers=12, num_heads=12,
                                 intermediate_size=1536, pooling="mean", max_seq_length=512,
                                 query_prefix="query: "),
    "bge-small-en-v1.5": EncoderConfig("bge-small-en-v1.5", hidden_size=384, num_layers=12, num_heads=12,
                                       intermediate_size=1536, pooling="cls", max_seq_length=512),
    "bge-base-en-v1.5": EncoderConfig("bge-base-en-v1.5", hidden_size=768, num_layers=12, num_heads=12,
                                      intermediate_size=3072, pooling="cls", max_seq_length=512),
    "bge-large-en-v1.5": EncoderConfig("bge-large-en-v1.5", hidden_size=1024, num_layers=24, num_heads=16,
                                       intermediate_size=4096, pooling="cls", max_seq_length=512),
    "encoder-tiny": EncoderConfig("encoder-tiny", vocab_size=2048, hidden_size=128, num_layers=2, num_heads=4,
                                  intermediate_size=256, max_position=256, max_seq_length=128),
}

ALIASES = {
    "qwen/qwen2.5-coder-7b-instruct-awq": "qwen2.5-coder-7b",
    "qwen/qwen2.5-coder-7b-instruct": "qwen2.5-coder-7b",
    "qwen/qwen2.5-3b-instruct": "qwen2.5-3b",
    "qwen/qwen2-7b": "qwen2-7b",
    "qwen/qwen2-7b-instruct": "qwen2-7b",
    "qwen/qwen2-1.5b": "qwen2-1.5b",
    "qwen/qwen2-72b": "qwen2-72b",
    "openai-community/gpt2": "gpt2",
    "openai-community/gpt2-medium": "gpt2-medium",
    "gpt2-small": "gpt2",
    "sentence-transformers/all-minilm-l6-v2": "all-minilm-l6-v2",
    "intfloat/e5-small-v2": "e5-small-v2",
    "baai/bge-base-en-v1.5": "bge-base-en-v1.5",
    "baai/bge-large-en-v1.5": "bge-large-en-v1.5",
    "baai/bge-small-en-v1.5": "bge-small-en-v1.5",
}


def _key(name: str) -> str:
    k = name.strip().lower()
    return ALIASES.get(k, k.split("/")[-1])


def decoder_config(name: str, **overrides):
    k = _key(name)
    cfg = HYBRIDS[k] if k in HYBRIDS else DECODERS[k]
    return replace(cfg, **overrides) if overrides else cfg


def encoder_config(name: str, **overrides) -> EncoderConfig:
    cfg = ENCODERS[_key(name)]
    return replace(cfg, **overrides) if overrides else cfg
