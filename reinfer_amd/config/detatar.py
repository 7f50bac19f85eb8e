"""Detatar: typed configuration from its config.json.

A decoder of parallel layers: one RMS norm in groups, and both the mixer and the feed-forward read its output;
the mixer reads it shifted towards the token before (a stored factor a channel), and each part's result enters
the residual stream times a sigmoid gate computed from the normed row. A layer's mixer is attention over a cached
low-rank latent whose queries go through a latent of their own, with one sigmoid gate a head
("latent_attention"), or a per-head matrix state with an input-dependent decay a key channel ("wkv"). Its
feed-forward is a gated dense one (the tanh form of gelu), a mixture of gated experts (softmax scores, a
correction that only the choice sees, groups of neighbours scored by their best member, identity experts, a
shared expert behind a sigmoid) or absent. A layer may use the tensors of an earlier layer (``weights_of``) with
a cache and state of its own. The embedding is scaled on its way in; the head is a tensor of its own.

config.json nests its keys: ``vocab``, ``width``, ``norm.{eps, groups}``, ``embedding.scale`` and ``layers[i]``
with ``type``, ``mixer``, ``mlp`` and, optionally, ``weights_of``. Tensor names: ``embed``, ``head``,
``final.norm``, ``l<i>.norm1``, ``l<i>.shift``, ``l<i>.rg1``, ``l<i>.rg1.b``, ``l<i>.rg2``, ``l<i>.rg2.b``,
``l<i>.mix.*``, ``l<i>.mlp.*``.
"""
from __future__ import annotations

from dataclasses import dataclass
from typing import Any, Dict, List, Mapping, Optional, Tuple, Union

from .puresun import _At, _section
from .schema import (BlockSpec, ConfigError, FeedForwardSpec, LatentAttentionSpec, MixerSpec, ModelSpec, MoESpec,
                     NormSpec, ParallelSpec, PositionSpec, RunEntry, WKVSpec, read_int)

ARCHITECTURE = "Detatar"

# config.json gives no context limit; the engine's own (block tables and captured steps are sized by it)
DEFAULT_MAX_POSITIONS = 1 << 16

# constants the design fixes
ROUTER_NORM_EPS = 1e-20         # added to the sum of the chosen scores before they are divided by it
GROUP_SCORE_TOP = 1             # a group of experts is scored by its largest choice score


@dataclass(frozen=True)
class DetatarLatentMixer:
    heads: int
    dim: int            # unrotated query/key entries a head
    rot_dim: int        # rotated query/key entries a head (one key part shared by all heads)
    vdim: int
    kv_rank: int
    q_rank: int
    scale: float
    rot_base: float
    rot_dims: int       # entries of the rotated part that are turned


@dataclass(frozen=True)
class DetatarWKVMixer:
    heads: int
    dim: int


@dataclass(frozen=True)
class DetatarDense:
    ff: int


@dataclass(frozen=True)
class DetatarMoE:
    experts: int
    identity: int
    top: int
    ff: int
    groups: int
    keep: int
    shared_ff: int          # 0: no shared expert


@dataclass(frozen=True)
class DetatarLayer:
    kind: str                                   # "latent_attention" or "wkv"
    mixer: Union[DetatarLatentMixer, DetatarWKVMixer]
    mlp: Union[DetatarDense, DetatarMoE, None]
    weights_of: Optional[int] = None            # the layer whose tensors this one uses (None: its own)


@dataclass(frozen=True)
class DetatarConfig:
    vocab: int
    width: int
    norm_eps: float
    norm_groups: int
    embedding_scale: float
    layers: Tuple[DetatarLayer, ...]
    decay_ranks: Tuple[int, ...] = ()           # rows of a wkv layer's first decay matrix, layer by layer (0: none)
    max_positions: int = DEFAULT_MAX_POSITIONS
    architecture: str = ARCHITECTURE

    # ---------------------------------------------------------------- reading
    @classmethod
    def from_dict(cls, cfg: Mapping[str, Any]) -> "DetatarConfig":
        vocab = read_int(cfg, "vocab", minimum=1)
        width = read_int(cfg, "width", minimum=1)
        nat = _At(_section(cfg, "norm"), "norm.")
        eps = nat.float("eps")
        if eps < 0.0:
            raise ConfigError("norm.eps", "must be >= 0")
        groups = nat.int("groups", 1, minimum=1)
        if width % groups:
            raise ConfigError("norm.groups", f"width {width} in {groups} equal groups")
        emb = _section(cfg, "embedding", required=False)
        emb_scale = _At(emb, "embedding.").float("scale", 1.0) if emb is not None else 1.0
        raw_layers = cfg.get("layers", None)
        if not isinstance(raw_layers, list) or not raw_layers:
            raise ConfigError("layers", "expected a non-empty list of layers")
        layers = tuple(cls._read_layer(L, f"layers[{i}].", i) for i, L in enumerate(raw_layers))
        for i, L in enumerate(layers):
            j = L.weights_of
            if j is not None:
                if layers[j].weights_of is not None:
                    raise ConfigError(f"layers[{i}].weights_of", f"layer {j} has no tensors of its own")
                if (layers[j].kind, layers[j].mixer, layers[j].mlp) != (L.kind, L.mixer, L.mlp):
                    raise ConfigError(f"layers[{i}].weights_of", f"the entry differs from layer {j}'s")
        ranks = cfg.get("decay_ranks", None)
        if ranks is None:
            ranks = ()
        elif not (isinstance(ranks, list) and len(ranks) == len(layers)
                  and all(isinstance(r, int) and not isinstance(r, bool) and r >= 0 for r in ranks)):
            raise ConfigError("decay_ranks", "expected one non-negative integer a layer")
        max_pos = read_int(cfg, "max_positions", DEFAULT_MAX_POSITIONS, minimum=1)
        return cls(vocab=vocab, width=width, norm_eps=eps, norm_groups=groups, embedding_scale=emb_scale,
                   layers=layers, decay_ranks=tuple(ranks), max_positions=max_pos)

    @staticmethod
    def _read_latent(m: Mapping[str, Any], where: str) -> DetatarLatentMixer:
        at = _At(m, where)
        heads, dim = at.int("heads", minimum=1), at.int("dim", minimum=0)
        rot_dim, vdim = at.int("rot_dim", minimum=0), at.int("vdim", minimum=1)
        if dim + rot_dim == 0:
            raise ConfigError(where + "dim", "a head needs at least one query/key entry")
        rot = _section(m, "rot", where, required=rot_dim > 0)
        base, dims = 10000.0, 0
        if rot is not None:
            rat = _At(rot, where + "rot.")
            base, dims = rat.float("base"), rat.int("dims", rot_dim, minimum=0)
            if base <= 0.0:
                raise ConfigError(where + "rot.base", "must be > 0")
            if dims % 2 or dims > rot_dim:
                raise ConfigError(where + "rot.dims", f"{dims} entries in pairs out of {rot_dim}")
        return DetatarLatentMixer(heads=heads, dim=dim, rot_dim=rot_dim, vdim=vdim,
                                  kv_rank=at.int("kv_rank", minimum=1), q_rank=at.int("q_rank", minimum=1),
                                  scale=at.float("scale"), rot_base=base, rot_dims=dims)

    @classmethod
    def _read_layer(cls, L: Any, where: str, index: int) -> DetatarLayer:
        if not isinstance(L, dict):
            raise ConfigError(where.rstrip("."), f"expected an object, got {L!r}")
        kind = L.get("type", None)
        m = _section(L, "mixer", where)
        if kind == "latent_attention":
            mixer: Any = cls._read_latent(m, where + "mixer.")
        elif kind == "wkv":
            at = _At(m, where + "mixer.")
            mixer = DetatarWKVMixer(heads=at.int("heads", minimum=1), dim=at.int("dim", minimum=1))
        else:
            raise ConfigError(where + "type", f"unknown mixer {kind!r}; this design has 'latent_attention' and 'wkv'")
        mlp: Any = None
        f = L.get("mlp", None)
        if f is not None:
            if not isinstance(f, dict):
                raise ConfigError(where + "mlp", f"expected an object or null, got {f!r}")
            fk = f.get("kind", None)
            if fk == "dense":
                mlp = DetatarDense(ff=_At(f, where + "mlp.").int("ff", minimum=1))
            elif fk == "moe":
                rsec = _section(f, "router", where + "mlp.")
                router = _At(rsec, where + "mlp.router.")
                experts, top = router.int("experts", minimum=1), router.int("top", minimum=1)
                identity = router.int("identity", 0, minimum=0)
                groups, keep = 1, 1
                gsec = _section(rsec, "groups", where + "mlp.router.", required=False)
                if gsec is not None:
                    gat = _At(gsec, where + "mlp.router.groups.")
                    groups, keep = gat.int("count", minimum=1), gat.int("keep", minimum=1)
                routed = experts + identity
                if routed % groups:
                    raise ConfigError(where + "mlp.router.groups.count",
                                      f"{routed} experts and identity experts in {groups} equal groups")
                if keep > groups:
                    raise ConfigError(where + "mlp.router.groups.keep", f"{keep} of {groups} groups")
                if top > keep * (routed // groups):
                    raise ConfigError(where + "mlp.router.top", f"{top} of the {keep * (routed // groups)} experts "
                                                                "that can be chosen")
                ff = _At(_section(f, "expert", where + "mlp."), where + "mlp.expert.").int("ff", minimum=1)
                ssec = _section(f, "shared", where + "mlp.", required=False)
                shared = _At(ssec, where + "mlp.shared.").int("ff", minimum=1) if ssec is not None else 0
                mlp = DetatarMoE(experts=experts, identity=identity, top=top, ff=ff, groups=groups, keep=keep,
                                 shared_ff=shared)
            else:
                raise ConfigError(where + "mlp.kind", f"unknown feed-forward {fk!r}; this design has 'dense' and 'moe'")
        src = L.get("weights_of", None)
        if src is not None:
            if isinstance(src, bool) or not isinstance(src, int) or not 0 <= src < index:
                raise ConfigError(where + "weights_of", f"expected the number of an earlier layer, got {src!r}")
        return DetatarLayer(kind=kind, mixer=mixer, mlp=mlp, weights_of=src)

    # ---------------------------------------------------------------- writing
    def to_dict(self) -> Dict[str, Any]:
        layers: List[Dict[str, Any]] = []
        for L in self.layers:
            m = L.mixer
            if L.kind == "wkv":
                mixer: Dict[str, Any] = {"dim": m.dim, "heads": m.heads}
            else:
                mixer = {"dim": m.dim, "heads": m.heads, "kv_rank": m.kv_rank, "q_rank": m.q_rank,
                         "rot_dim": m.rot_dim, "scale": m.scale, "vdim": m.vdim}
                if m.rot_dim:
                    mixer["rot"] = {"base": m.rot_base, "dims": m.rot_dims}
            mlp: Any = None
            if isinstance(L.mlp, DetatarDense):
                mlp = {"ff": L.mlp.ff, "kind": "dense"}
            elif isinstance(L.mlp, DetatarMoE):
                f = L.mlp
                mlp = {"expert": {"ff": f.ff}, "kind": "moe",
                       "router": {"experts": f.experts, "groups": {"count": f.groups, "keep": f.keep},
                                  "identity": f.identity, "top": f.top}}
                if f.shared_ff:
                    mlp["shared"] = {"ff": f.shared_ff}
            entry: Dict[str, Any] = {"mixer": mixer, "mlp": mlp, "type": L.kind}
            if L.weights_of is not None:
                entry["weights_of"] = L.weights_of
            layers.append(entry)
        d: Dict[str, Any] = {"architecture": ARCHITECTURE, "embedding": {"scale": self.embedding_scale},
                             "layers": layers, "norm": {"eps": self.norm_eps, "groups": self.norm_groups},
                             "vocab": self.vocab, "width": self.width}
        if any(self.decay_ranks):
            d["decay_ranks"] = list(self.decay_ranks)
        if self.max_positions != DEFAULT_MAX_POSITIONS:
            d["max_positions"] = self.max_positions
        return d

    # ---------------------------------------------------------------- the model
    def with_tensor_shapes(self, shapes: Mapping[str, Tuple[int, ...]]) -> "DetatarConfig":
        """The configuration with the sizes that only the tensors give: the rank of a wkv layer's decay, the
        rows of ``l<i>.mix.w1``."""
        ranks = []
        for i, L in enumerate(self.layers):
            shape = shapes.get(f"l{i}.mix.w1") if L.kind == "wkv" and L.weights_of is None else None
            ranks.append(int(shape[0]) if shape is not None else 0)
        return DetatarConfig(**{**self.__dict__, "decay_ranks": tuple(ranks)})

    def _decay_rank(self, i: int) -> int:
        r = self.decay_ranks[i] if i < len(self.decay_ranks) else 0
        if r <= 0:
            raise ConfigError(f"layers[{i}].mixer", "the rank of the decay is the number of rows of the layer's "
                                                    "mix.w1 tensor: read it with with_tensor_shapes(), or give "
                                                    "decay_ranks")
        return r

    def _mixer_spec(self, i: int, L: DetatarLayer) -> MixerSpec:
        m = L.mixer
        if L.kind == "wkv":
            return MixerSpec(kind="wkv", hidden=self.width,
                             params=WKVSpec(heads=m.heads, dim=m.dim, decay_rank=self._decay_rank(i),
                                            norm_eps=self.norm_eps))
        return MixerSpec(
            kind="latent_attention", hidden=self.width, num_heads=m.heads, num_kv_heads=1, head_dim=m.dim,
            scale=m.scale, window=0,
            position=PositionSpec("rope_neox", rotary_dim=m.rot_dims, theta=m.rot_base) if m.rot_dims
            else PositionSpec("none"),
            params=LatentAttentionSpec(rank=m.kv_rank, rot_width=m.rot_dim, value_dim=m.vdim, norm_eps=self.norm_eps,
                                       gated=True, head_gate=True, q_rank=m.q_rank))

    def _ffn_spec(self, f) -> Optional[FeedForwardSpec]:
        if f is None:
            return None
        if isinstance(f, DetatarDense):
            return FeedForwardSpec(kind="swiglu", hidden=self.width, intermediate=f.ff,
                                   extra=(("names", ("gate", "up", "down")), ("act", "gelu_tanh")))
        return FeedForwardSpec(kind="moe", hidden=self.width, intermediate=f.ff,
                               params=MoESpec(experts=f.experts, top=f.top, activation="silu_gated", weights="softmax",
                                              groups=f.groups, groups_kept=f.keep, group_top=GROUP_SCORE_TOP,
                                              shared=f.shared_ff, identity=f.identity, correction=True,
                                              norm_eps=ROUTER_NORM_EPS, shared_gated=f.shared_ff > 0))

    def to_spec(self) -> ModelSpec:
        norm = NormSpec("rmsnorm", self.width, self.norm_eps, groups=self.norm_groups)
        blocks: List[BlockSpec] = []
        block_of: Dict[int, int] = {}
        order: List[RunEntry] = []
        for i, L in enumerate(self.layers):
            if L.weights_of is None:
                block_of[i] = len(blocks)
                blocks.append(BlockSpec(kind="parallel", mixer=self._mixer_spec(i, L), ffn=self._ffn_spec(L.mlp),
                                        mixer_norm=norm, prefix=f"l{i}.", mixer_prefix="mix.", ffn_prefix="mlp.",
                                        mixer_norm_name="norm1",
                                        params=ParallelSpec(token_shift=True, gated=True, shift_name="shift",
                                                            gate_names=("rg1", "rg2"))))
            # a layer that uses another's tensors runs that layer's block again, with a cache and state of its own
            order.append(RunEntry(block_of[L.weights_of if L.weights_of is not None else i]))
        return ModelSpec(
            architecture=ARCHITECTURE, vocab_size=self.vocab, hidden=self.width, max_positions=self.max_positions,
            blocks=tuple(blocks), run_order=tuple(order), final_norm=norm, tie_embeddings=False,
            embed_name="embed", final_norm_name="final.norm", head_name="head", embed_scale=self.embedding_scale)
