"""Gibavik: typed configuration from its config.json.

A decoder whose sublayers read the residual stream itself and whose results enter it behind an RMS norm with one
number for all coordinates: x <- x + norm1(mixer(x)), x <- x + norm2(ff(x)). A layer's mixer is grouped-query
attention with biases, queries and keys normed over their whole projection, no rotation and a logarithmic
distance term a head taken off the scores ("attention"; such a layer may read the keys and values of an earlier
layer, ``kv_from``), or two mixers side by side added up with a constant each ("parallel": attention inside a
sliding window with per-head query/key norm, rotation of part of a head, values that turn with their position,
scores capped by a tanh and a sigmoid gate on the heads; and a matrix memory a head that fades by a constant).
Its feed-forward is a gated dense one with bounded inputs, a mixture of gated experts that a table gives each
token id, or absent. The embedding is scaled on its way in, the head is a tensor of its own and the logits are
capped by a tanh.

config.json nests its keys: ``vocab``, ``width``, ``norm.eps``, ``embedding.scale``, ``logit_softcap`` and
``layers[i]`` with ``type``, ``mixer`` and ``mlp``. Tensor names: ``embed``, ``head``, ``final.norm``,
``l<i>.norm1``, ``l<i>.norm2``, ``l<i>.mix.*`` (``.left.*`` / ``.right.*`` in a parallel layer), ``l<i>.mlp.*``.
What a model may leave out means "not there": no window, no rotation (and then no turning of the values), no cap,
a scale of 1 / sqrt(size), factors of 1.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, List, Mapping, Optional, Tuple, Union

from .puresun import _At, _section
from .schema import (BlockSpec, ConfigError, DecayMemorySpec, FeedForwardSpec, MixerSpec, ModelSpec, MoESpec,
                     NormSpec, PositionSpec, RunEntry, SideBySideSpec, read_float, read_int)

ARCHITECTURE = "Gibavik"

# config.json gives no context limit; the engine's own (block tables and captured steps are sized by it)
DEFAULT_MAX_POSITIONS = 1 << 16


@dataclass(frozen=True)
class GibavikAttention:
    """Either attention of the design; ``windowed`` picks the form of the side-by-side layer's left mixer."""
    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    window: int = 0             # 0: every earlier key
    rot_base: float = 10000.0
    rot_dims: int = 0           # 0: no rotation
    softcap: float = 0.0        # 0: none
    kv_from: Optional[int] = None


@dataclass(frozen=True)
class GibavikMemory:
    heads: int
    dim: int
    vdim: int
    decay: Tuple[float, ...]


@dataclass(frozen=True)
class GibavikPair:
    left: GibavikAttention
    right: GibavikMemory
    left_scale: float
    right_scale: float


@dataclass(frozen=True)
class GibavikDense:
    ff: int
    limit: float


@dataclass(frozen=True)
class GibavikMoE:
    experts: int
    top: int
    ff: int


@dataclass(frozen=True)
class GibavikLayer:
    kind: str                                   # "attention" or "parallel"
    mixer: Union[GibavikAttention, GibavikPair]
    mlp: Union[GibavikDense, GibavikMoE, None]


@dataclass(frozen=True)
class GibavikConfig:
    vocab: int
    width: int
    norm_eps: float
    embedding_scale: float
    logit_softcap: float
    layers: Tuple[GibavikLayer, ...]
    max_positions: int = DEFAULT_MAX_POSITIONS
    architecture: str = ARCHITECTURE

    # ---------------------------------------------------------------- reading
    @classmethod
    def from_dict(cls, cfg: Mapping[str, Any]) -> "GibavikConfig":
        vocab = read_int(cfg, "vocab", minimum=1)
        width = read_int(cfg, "width", minimum=1)
        eps = _At(_section(cfg, "norm"), "norm.").float("eps")
        if eps < 0.0:
            raise ConfigError("norm.eps", "must be >= 0")
        emb = _section(cfg, "embedding", required=False)
        emb_scale = _At(emb, "embedding.").float("scale", 1.0) if emb is not None else 1.0
        cap = read_float(cfg, "logit_softcap", 0.0)
        if cap < 0.0:
            raise ConfigError("logit_softcap", "must be >= 0 (absent: no cap)")
        raw_layers = cfg.get("layers", None)
        if not isinstance(raw_layers, list) or not raw_layers:
            raise ConfigError("layers", "expected a non-empty list of layers")
        layers = tuple(cls._read_layer(L, f"layers[{i}].") for i, L in enumerate(raw_layers))
        for i, L in enumerate(layers):
            src = L.mixer.kv_from if L.kind == "attention" else None
            if src is None:
                continue
            where = f"layers[{i}].mixer.kv_from"
            if not 0 <= src < i:
                raise ConfigError(where, f"layer {src} must come before layer {i}")
            S = layers[src]
            if S.kind != "attention" or S.mixer.kv_from is not None:
                raise ConfigError(where, f"layer {src} keeps no keys and values of its own for an attention layer to read")
            a, b = L.mixer, S.mixer
            if (a.kv_heads, a.dim, a.vdim, a.window) != (b.kv_heads, b.dim, b.vdim, b.window):
                raise ConfigError(where, f"layer {src} keeps other heads or another window than layer {i} reads")
        max_pos = read_int(cfg, "max_positions", DEFAULT_MAX_POSITIONS, minimum=1)
        return cls(vocab=vocab, width=width, norm_eps=eps, embedding_scale=emb_scale, logit_softcap=cap,
                   layers=layers, max_positions=max_pos)

    @staticmethod
    def _read_attention(m: Mapping[str, Any], where: str, may_share: bool) -> GibavikAttention:
        at = _At(m, where)
        heads, kv = at.int("heads", minimum=1), at.int("kv_heads", minimum=1)
        if heads % kv:
            raise ConfigError(where + "kv_heads", f"{heads} query heads do not divide into {kv} groups")
        dim, vdim = at.int("dim", minimum=1), at.int("vdim", minimum=1)
        mask = _section(m, "mask", where, required=False)
        window = _At(mask, where + "mask.").int("size", minimum=1) if mask is not None else 0
        rot = _section(m, "rot", where, required=False)
        base, dims = 10000.0, 0
        if rot is not None:
            rat = _At(rot, where + "rot.")
            base, dims = rat.float("base"), rat.int("dims", minimum=0)
            if base <= 0.0:
                raise ConfigError(where + "rot.base", "must be > 0")
            if dims % 2 or dims > dim:
                raise ConfigError(where + "rot.dims", f"{dims} entries in pairs out of {dim}")
            if dims and vdim % 2:
                raise ConfigError(where + "vdim", f"values of {vdim} entries do not turn in pairs")
        cap = at.float("softcap", 0.0)
        if cap < 0.0:
            raise ConfigError(where + "softcap", "must be > 0 (absent: no cap)")
        src = m.get("kv_from", None)
        if src is not None:
            if not may_share:
                raise ConfigError(where + "kv_from", "only an attention layer reads another layer's keys and values")
            src = at.int("kv_from", minimum=0)
        return GibavikAttention(heads=heads, kv_heads=kv, dim=dim, vdim=vdim,
                                scale=at.float("scale", float(dim) ** -0.5), window=window, rot_base=base,
                                rot_dims=dims, softcap=cap, kv_from=src)

    @staticmethod
    def _read_memory(m: Mapping[str, Any], where: str) -> GibavikMemory:
        at = _At(m, where)
        heads = at.int("heads", minimum=1)
        decay = m.get("decay", None)
        if not isinstance(decay, list) or len(decay) != heads or \
                any(isinstance(d, bool) or not isinstance(d, (int, float)) for d in decay):
            raise ConfigError(where + "decay", f"expected {heads} numbers, one a head")
        return GibavikMemory(heads=heads, dim=at.int("dim", minimum=1), vdim=at.int("vdim", minimum=1),
                             decay=tuple(float(d) for d in decay))

    @classmethod
    def _read_layer(cls, L: Any, where: str) -> GibavikLayer:
        if not isinstance(L, dict):
            raise ConfigError(where.rstrip("."), f"expected an object, got {L!r}")
        kind = L.get("type", None)
        m = _section(L, "mixer", where)
        if kind == "attention":
            mixer: Any = cls._read_attention(m, where + "mixer.", True)
        elif kind == "parallel":
            at = _At(m, where + "mixer.")
            mixer = GibavikPair(
                left=cls._read_attention(_section(m, "left", where + "mixer."), where + "mixer.left.", False),
                right=cls._read_memory(_section(m, "right", where + "mixer."), where + "mixer.right."),
                left_scale=at.float("left_scale", 1.0), right_scale=at.float("right_scale", 1.0))
        else:
            raise ConfigError(where + "type", f"unknown mixer {kind!r}; this design has 'attention' and 'parallel'")
        mlp: Any = None
        f = L.get("mlp", None)
        if f is not None:
            if not isinstance(f, dict):
                raise ConfigError(where + "mlp", f"expected an object or null, got {f!r}")
            fk = f.get("kind", None)
            if fk == "dense":
                fat = _At(f, where + "mlp.")
                limit = fat.float("limit")
                if not limit > 0.0:
                    raise ConfigError(where + "mlp.limit", "must be > 0")
                mlp = GibavikDense(ff=fat.int("ff", minimum=1), limit=limit)
            elif fk == "moe":
                router = _At(_section(f, "router", where + "mlp."), where + "mlp.router.")
                experts, top = router.int("experts", minimum=1), router.int("top", minimum=1)
                if top > experts:
                    raise ConfigError(where + "mlp.router.top", f"{top} different experts of {experts}")
                ff = _At(_section(f, "expert", where + "mlp."), where + "mlp.expert.").int("ff", minimum=1)
                mlp = GibavikMoE(experts=experts, top=top, ff=ff)
            else:
                raise ConfigError(where + "mlp.kind", f"unknown feed-forward {fk!r}; this design has 'dense' and 'moe'")
        return GibavikLayer(kind=kind, mixer=mixer, mlp=mlp)

    # ---------------------------------------------------------------- writing
    @staticmethod
    def _attention_dict(a: GibavikAttention) -> Dict[str, Any]:
        d: Dict[str, Any] = {"dim": a.dim, "heads": a.heads, "kv_heads": a.kv_heads, "scale": a.scale, "vdim": a.vdim}
        if a.window:
            d["mask"] = {"size": a.window}
        if a.rot_dims:
            d["rot"] = {"base": a.rot_base, "dims": a.rot_dims}
        if a.softcap:
            d["softcap"] = a.softcap
        if a.kv_from is not None:
            d["kv_from"] = a.kv_from
        return d

    def to_dict(self) -> Dict[str, Any]:
        layers: List[Dict[str, Any]] = []
        for L in self.layers:
            if L.kind == "attention":
                mixer = self._attention_dict(L.mixer)
            else:
                r = L.mixer.right
                mixer = {"left": self._attention_dict(L.mixer.left), "left_scale": L.mixer.left_scale,
                         "right": {"decay": list(r.decay), "dim": r.dim, "heads": r.heads, "vdim": r.vdim},
                         "right_scale": L.mixer.right_scale}
            mlp: Any = None
            if isinstance(L.mlp, GibavikDense):
                mlp = {"ff": L.mlp.ff, "kind": "dense", "limit": L.mlp.limit}
            elif isinstance(L.mlp, GibavikMoE):
                mlp = {"expert": {"ff": L.mlp.ff}, "kind": "moe",
                       "router": {"experts": L.mlp.experts, "top": L.mlp.top}}
            layers.append({"mixer": mixer, "mlp": mlp, "type": L.kind})
        d: Dict[str, Any] = {"architecture": ARCHITECTURE, "embedding": {"scale": self.embedding_scale},
                             "layers": layers, "norm": {"eps": self.norm_eps}, "vocab": self.vocab,
                             "width": self.width}
        if self.logit_softcap:
            d["logit_softcap"] = self.logit_softcap
        if self.max_positions != DEFAULT_MAX_POSITIONS:
            d["max_positions"] = self.max_positions
        return d

    # ---------------------------------------------------------------- the model
    _NAMES = (("names", ("q", "k", "v", "o")), ("bias_suffix", ".b"), ("norm_names", ("q.norm", "k.norm")))

    def _attention_spec(self, a: GibavikAttention, windowed: bool) -> MixerSpec:
        if windowed:
            # the side-by-side layer's left mixer: per-head norm, rotation, turning values, cap, window, gate
            return MixerSpec(kind="gqa_attention", hidden=self.width, num_heads=a.heads, num_kv_heads=a.kv_heads,
                             head_dim=a.dim, value_dim=a.vdim, scale=a.scale, window=a.window, qk_norm=True,
                             qk_norm_eps=self.norm_eps, bias=True,
                             position=PositionSpec("rope_neox", rotary_dim=a.rot_dims, theta=a.rot_base)
                             if a.rot_dims else PositionSpec("none"),
                             extra=self._NAMES, softcap=a.softcap, rotate_values=a.rot_dims > 0, out_gate=True)
        return MixerSpec(kind="gqa_attention", hidden=self.width, num_heads=a.heads, num_kv_heads=a.kv_heads,
                         head_dim=a.dim, value_dim=a.vdim, scale=a.scale, window=a.window, qk_norm_eps=self.norm_eps,
                         bias=True, extra=self._NAMES, qk_norm_whole=True, softcap=a.softcap, distance_bias=True,
                         kv_shared=a.kv_from is not None)

    def _mixer_spec(self, L: GibavikLayer) -> MixerSpec:
        if L.kind == "attention":
            return self._attention_spec(L.mixer, False)
        r = L.mixer.right
        right = MixerSpec(kind="decay_memory", hidden=self.width,
                          params=DecayMemorySpec(heads=r.heads, key_dim=r.dim, value_dim=r.vdim, decays=r.decay,
                                                 norm_eps=self.norm_eps))
        return MixerSpec(kind="side_by_side", hidden=self.width,
                         params=SideBySideSpec(members=(("left.", self._attention_spec(L.mixer.left, True)),
                                                        ("right.", right)),
                                               norm_eps=self.norm_eps, combine="scaled_sum",
                                               scales=(L.mixer.left_scale, L.mixer.right_scale)))

    def _ffn_spec(self, f) -> Optional[FeedForwardSpec]:
        if f is None:
            return None
        if isinstance(f, GibavikDense):
            return FeedForwardSpec(kind="swiglu", hidden=self.width, intermediate=f.ff,
                                   extra=(("names", ("gate", "up", "down")), ("act", "swish_bounded"),
                                          ("limit", f.limit)))
        return FeedForwardSpec(kind="moe", hidden=self.width, intermediate=f.ff, extra=(("vocab", self.vocab),),
                               params=MoESpec(experts=f.experts, top=f.top, activation="silu_gated", weights="table"))

    def to_spec(self) -> ModelSpec:
        norm = NormSpec("rmsnorm", self.width, self.norm_eps, scalar=True)
        blocks: List[BlockSpec] = []
        order: List[RunEntry] = []
        for i, L in enumerate(self.layers):
            ffn = self._ffn_spec(L.mlp)
            blocks.append(BlockSpec(kind="outnorm", mixer=self._mixer_spec(L), ffn=ffn, mixer_norm=norm,
                                    ffn_norm=norm if ffn is not None else None, prefix=f"l{i}.",
                                    mixer_prefix="mix.", ffn_prefix="mlp.", mixer_norm_name="norm1",
                                    ffn_norm_name="norm2"))
            src = L.mixer.kv_from if L.kind == "attention" else None
            order.append(RunEntry(i, cache_from=src))
        return ModelSpec(
            architecture=ARCHITECTURE, vocab_size=self.vocab, hidden=self.width, max_positions=self.max_positions,
            blocks=tuple(blocks), run_order=tuple(order), final_norm=norm, tie_embeddings=False,
            embed_name="embed", final_norm_name="final.norm", head_name="head", embed_scale=self.embedding_scale,
            logit_softcap=self.logit_softcap)
