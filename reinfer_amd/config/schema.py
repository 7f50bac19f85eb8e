"""Typed descriptions of a model: what the parts are built from.

A configuration class (one per architecture) reads the architecture's own
``config.json`` keys and turns them into a :class:`ModelSpec`: a list of
blocks, each naming its mixer, feed-forward, norms and position encoding with
every size and constant as a field, plus the order in which the blocks run.
Parts are built from these records alone; none of them knows which model it
belongs to.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Dict, List, Mapping, Optional, Tuple


class ConfigError(ValueError):
    """A config.json key is missing or holds a value the engine cannot run.

    ``key`` names the offending key (the reference's ``ArchError::MissingKey``
    / ``InvalidValue`` carry the key the same way,
    crates/arch/src/llama.rs:122-173).
    """

    def __init__(self, key: str, why: str):
        super().__init__(f"config.json: {key}: {why}")
        self.key = key
        self.why = why


class UnknownArchitecture(ConfigError):
    def __init__(self, name: str, known: List[str]):
        ValueError.__init__(
            self, f"config.json: unknown architecture {name!r}; registered: {sorted(known)}")
        self.key = "architectures"
        self.why = "unknown architecture"
        self.name = name


# --------------------------------------------------------------------------
# key readers (fail closed, error names the key)
# --------------------------------------------------------------------------

_MISSING = object()


def read_int(cfg: Mapping[str, Any], key: str, default: Any = _MISSING, *, minimum: int = 0) -> int:
    v = cfg.get(key, None)
    if v is None:
        if default is _MISSING:
            raise ConfigError(key, "required key is missing")
        return default
    if isinstance(v, bool) or not isinstance(v, int):
        if isinstance(v, float) and float(v).is_integer():
            v = int(v)
        else:
            raise ConfigError(key, f"expected an integer, got {v!r}")
    if v < minimum:
        raise ConfigError(key, f"must be >= {minimum}, got {v}")
    return int(v)


def read_float(cfg: Mapping[str, Any], key: str, default: Any = _MISSING) -> float:
    v = cfg.get(key, None)
    if v is None:
        if default is _MISSING:
            raise ConfigError(key, "required key is missing")
        return default
    if isinstance(v, bool) or not isinstance(v, (int, float)):
        raise ConfigError(key, f"expected a number, got {v!r}")
    v = float(v)
    if v != v or v in (float("inf"), float("-inf")):
        raise ConfigError(key, "must be finite")
    return v


def read_bool(cfg: Mapping[str, Any], key: str, default: bool) -> bool:
    v = cfg.get(key, None)
    if v is None:
        return default
    if not isinstance(v, bool):
        raise ConfigError(key, f"expected true/false, got {v!r}")
    return v


# --------------------------------------------------------------------------
# part specifications
# --------------------------------------------------------------------------

@dataclass(frozen=True)
class NormSpec:
    kind: str            # registry name of the norm part, e.g. "rmsnorm"
    size: int
    eps: float
    offset: float = 0.0  # the stored weight lies around zero: the factor is offset + w (1.0 for "one plus w")
    groups: int = 1      # the row is normed in this many equal consecutive parts, each over its own root mean square
    scalar: bool = False # the stored weight is one number that multiplies every coordinate


@dataclass(frozen=True)
class PositionSpec:
    kind: str            # e.g. "rope_neox"; "none" for no position encoding
    rotary_dim: int = 0
    theta: float = 10000.0
    extra: Tuple[Tuple[str, Any], ...] = ()   # for position parts defined elsewhere

    def option(self, name: str, default: Any = None) -> Any:
        return dict(self.extra).get(name, default)


@dataclass(frozen=True)
class MixerSpec:
    """Token mixer of a block. ``kind`` picks the part; fields are its sizes."""
    kind: str                       # e.g. "gqa_attention"
    hidden: int
    num_heads: int = 0
    num_kv_heads: int = 0
    head_dim: int = 0
    scale: float = 0.0              # multiplies q.k before softmax
    window: int = 0                 # 0: all earlier keys; W>0: the last W keys
    qk_norm: bool = False           # per-head norm of q and k before rotation
    qk_norm_eps: float = 1e-6
    bias: bool = False
    position: PositionSpec = PositionSpec("none")
    extra: Tuple[Tuple[str, Any], ...] = ()   # for mixers defined elsewhere
    value_dim: int = 0              # size of a value head where it differs from head_dim (0: the same)
    # A mixer that is not attention-shaped brings a record of its own (any frozen dataclass) with the
    # sizes and constants it needs, typed as it likes; the fields above then stay at their defaults.
    params: Any = None
    # further options of attention
    qk_norm_whole: bool = False     # q and k are normed over their whole projection (all heads at once), weights of that size
    softcap: float = 0.0            # score <- softcap * tanh(score / softcap) when > 0
    distance_bias: bool = False     # score -= r1_h * ln(1 + r2_h * (i - j)), two numbers a query head
    rotate_values: bool = False     # a value is turned by its own position over its whole size, a head's result back by the query's
    out_gate: bool = False          # the concatenated heads times sigmoid(W_g h), element by element, before the output projection
    kv_shared: bool = False         # the mixer has no key and value tensors: it reads another run entry's cache

    def option(self, name: str, default: Any = None) -> Any:
        return dict(self.extra).get(name, default)


@dataclass(frozen=True)
class FeedForwardSpec:
    kind: str                       # e.g. "swiglu"
    hidden: int
    intermediate: int
    extra: Tuple[Tuple[str, Any], ...] = ()
    params: Any = None              # a record of its own for a feed-forward defined elsewhere (experts, routing)


@dataclass(frozen=True)
class LatentAttentionSpec:
    """Sizes of an attention whose keys and values are linear maps of one cached latent vector a token
    (``MixerSpec.params`` of the "latent_attention" mixer; heads, scale, window and rotation are the
    ``MixerSpec``'s own fields): a query head is ``head_dim`` unrotated and ``rot_width`` rotated entries, the
    latent ``rank`` wide, a value head ``value_dim``; ``gated``: the concatenated heads are multiplied by the
    sigmoid of a projection of the mixer's input before the output projection, element by element, or, with
    ``head_gate``, by one number a head. ``q_rank`` > 0: the queries come through a latent of their own,
    q = W_uq rms(W_dq h) with a plain norm weight (0: q = W_q h)."""
    rank: int
    rot_width: int
    value_dim: int
    norm_eps: float
    gated: bool = True
    head_gate: bool = False
    q_rank: int = 0


@dataclass(frozen=True)
class MoESpec:
    """Routing of a mixture-of-experts feed-forward (``FeedForwardSpec.params``; ``intermediate`` is one
    expert's width): ``experts`` of which each token uses ``top``; ``activation`` of an expert ("relu2": the
    square of relu, no gate; "silu_gated": silu(gate) * up, an expert then has a gate matrix as well);
    ``weights``: "softmax_chosen" = softmax over the chosen logits alone; "sigmoid" = the sigmoid of each chosen
    logit times ``weight_scale``, not renormalised. ``groups`` > 1: the experts form that many equal runs of
    neighbours, a run's score is the sum of its ``group_top`` largest scores, and only experts of the
    ``groups_kept`` best runs can be chosen. ``shared`` > 0: one more expert of that width, same form, runs
    for every token with weight 1, or, with ``shared_gated``, times the sigmoid of one more router output.
    ``weights`` "softmax": scores are the softmax over all router outputs, the choice is by score plus a stored
    correction (``correction``) inside the best groups (``group_top`` 1: a group's score is its largest choice
    score), the weights the chosen scores over their sum + ``norm_eps``. ``identity`` > 0: that many further
    router outputs behind the experts stand for experts without matrices whose output is their input.
    ``weights`` "table": no router; an integer table [vocabulary, top] gives each token id its experts, each
    weighing 1 / top."""
    experts: int
    top: int
    activation: str = "relu2"
    weights: str = "softmax_chosen"
    weight_scale: float = 1.0
    groups: int = 1
    groups_kept: int = 1
    group_top: int = 2
    shared: int = 0
    identity: int = 0
    correction: bool = False
    norm_eps: float = 0.0
    shared_gated: bool = False


@dataclass(frozen=True)
class MatrixMemorySpec:
    """A matrix memory with exponential gates (``MixerSpec.params`` of the "matrix_memory" mixer): per head a
    [key_dim, value_dim] state, a normaliser vector and a running maximum of the log gates; the log input gate
    and the pre-activation of the forget gate are soft-capped at ``gate_cap`` (0: no cap); ``norm_eps`` is the
    eps of the per-head norm of the read-out; ``denom_eps`` is added to the read-out's denominator."""
    heads: int
    key_dim: int
    value_dim: int
    gate_cap: float
    norm_eps: float
    denom_eps: float = 1e-6


@dataclass(frozen=True)
class DecayMemorySpec:
    """A matrix state a head that fades by a constant a head (``MixerSpec.params`` of the "decay_memory" mixer):
    S <- decays[h] * S + k v^T, o = S^T q, with ``heads`` heads of ``key_dim`` x ``value_dim`` and silu on q, k and
    v; the concatenated read-outs are RMS-normed together (``norm_eps``), times a plain weight and a sigmoid
    gate."""
    heads: int
    key_dim: int
    value_dim: int
    decays: Tuple[float, ...]
    norm_eps: float


@dataclass(frozen=True)
class WKVSpec:
    """A matrix state a head with a decay a key channel that depends on the input (``MixerSpec.params`` of the
    "wkv" mixer): ``heads`` heads of ``dim`` x ``dim``; receptance, key, value, gate and decay each read their own
    mix of the input row with the row of the token before; the decay's pre-activation goes through a low-rank
    pair of ``decay_rank``; ``norm_eps`` is the eps of the per-head norm of the read-out."""
    heads: int
    dim: int
    decay_rank: int
    norm_eps: float


@dataclass(frozen=True)
class ParallelSpec:
    """Options of the "parallel" arrangement (``BlockSpec.params``). ``token_shift``: what the mixer reads is
    h + (h' - h) * s with h' the normed row of the token before (zeros for a request's first token, the last row
    kept in the request's state) and s the vector ``shift_name``. ``gated``: each part's result enters the
    stream times sigmoid(W h + b), W and b named by ``gate_names`` (mixer, feed-forward; the bias is the name
    plus ``.b``), h the normed row before any shift."""
    token_shift: bool = False
    gated: bool = False
    shift_name: str = "shift"
    gate_names: Tuple[str, str] = ("rg1", "rg2")


@dataclass(frozen=True)
class DeltaRuleSpec:
    """A gated delta rule (``MixerSpec.params`` of the "gated_delta_rule" mixer): ``heads`` value heads of
    ``value_dim``, ``key_heads`` query/key heads of ``key_dim`` shared by heads // key_heads value heads each, a
    causal filter of ``conv_taps`` taps over time on q, k and v, ``unit_eps`` inside the root of the unit norm
    of q and k, ``norm_eps`` of the per-head norm of the read-out."""
    heads: int
    key_heads: int
    key_dim: int
    value_dim: int
    conv_taps: int
    norm_eps: float
    unit_eps: float = 1e-6


@dataclass(frozen=True)
class SideBySideSpec:
    """Several mixers on one input (``MixerSpec.params`` of the "side_by_side" mixer): ``members`` are
    (tensor-name prefix, MixerSpec) pairs; each member's output is RMS-normed over the width (``norm_eps``) with
    a plain weight ``<prefix><out_name>`` and the results are averaged."""
    members: Tuple[Tuple[str, Any], ...]
    norm_eps: float
    out_name: str = "out"
    # "normed_mean" as above; "scaled_sum": y = sum_i scales[i] * mixer_i(h), no norms and no weights
    combine: str = "normed_mean"
    scales: Tuple[float, ...] = ()


@dataclass(frozen=True)
class InputSpec:
    """Something added to the token embedding before the first layer, beyond positions: ``kind`` picks the
    part (registry "input"), ``params`` is the part's own typed record, ``prefix`` goes before its tensor
    names."""
    kind: str
    params: Any = None
    prefix: str = ""


@dataclass(frozen=True)
class PairHashSpec:
    """A table of ``buckets`` + 1 rows looked up by a hash of (previous token, token):
    row = (previous * mul_prev + token * mul_cur) mod buckets; a request's first token takes the last row."""
    buckets: int
    mul_prev: int
    mul_cur: int
    table_name: str = "bigram"


@dataclass(frozen=True)
class StreamAdd:
    """What is added to the residual stream right before a run-order entry: the embedding output once more
    (``embedding``), and row ``row`` of the [rows, width] tensor ``vector`` (None: no vector)."""
    embedding: bool = False
    vector: Optional[str] = None
    row: int = 0


@dataclass(frozen=True)
class BlockSpec:
    """One layer: how norm, mixer and feed-forward are arranged, and its parts.

    The four part records are what the "prenorm" arrangement is built from; another arrangement may
    leave any of them out (one norm for both parts, a layer that only mixes) and bring a typed record
    of its own in ``params`` (any frozen dataclass), or loose options in ``extra``."""
    kind: str                       # e.g. "prenorm": x += mixer(norm(x)); x += ffn(norm(x))
    mixer: Optional[MixerSpec] = None
    ffn: Optional[FeedForwardSpec] = None
    mixer_norm: Optional[NormSpec] = None
    ffn_norm: Optional[NormSpec] = None
    prefix: str = ""                # tensor-name prefix of this block's weights
    mixer_prefix: str = "self_attn."
    ffn_prefix: str = "mlp."
    mixer_norm_name: str = "input_layernorm.weight"
    ffn_norm_name: str = "post_attention_layernorm.weight"
    residual_scale: float = 1.0     # x += residual_scale * part(norm(x)) for both parts of the block
    params: Any = None
    extra: Tuple[Tuple[str, Any], ...] = ()

    def option(self, name: str, default: Any = None) -> Any:
        return dict(self.extra).get(name, default)


@dataclass(frozen=True)
class RunEntry:
    """One position in the run order.

    ``block`` indexes ``ModelSpec.blocks`` (a block may appear more than once:
    shared weights, separate cache). ``cache_from`` names an earlier run entry
    whose cache this entry reads instead of keeping one of its own.
    """
    block: int
    cache_from: Optional[int] = None
    before: Optional[StreamAdd] = None      # added to the stream right before this entry runs


@dataclass(frozen=True)
class ModelSpec:
    architecture: str
    vocab_size: int
    hidden: int
    max_positions: int
    blocks: Tuple[BlockSpec, ...]
    run_order: Tuple[RunEntry, ...]
    final_norm: NormSpec
    tie_embeddings: bool
    embed_name: str = "model.embed_tokens.weight"
    final_norm_name: str = "model.norm.weight"
    head_name: str = "lm_head.weight"
    eos_token_ids: Tuple[int, ...] = ()
    bos_token_id: Optional[int] = None
    # a position encoding that is added to the embeddings (learned or computed absolute positions), for
    # architectures whose mixers do not rotate; None: positions enter in the mixers only
    input_position: Optional[PositionSpec] = None
    input_position_prefix: str = "model."
    # further parts that add to the embedding (a hashed token-pair table, ...), in order
    inputs: Tuple[InputSpec, ...] = ()
    # [rows, width] tensors whose rows run-order entries add to the stream (``RunEntry.before``): (name, rows)
    stream_vectors: Tuple[Tuple[str, int], ...] = ()
    # logits <- cap * tanh(logits / cap) when cap > 0
    logit_softcap: float = 0.0
    # the embedding rows are multiplied by this on their way into the stream (a tied head uses the table as it is)
    embed_scale: float = 1.0

    def __post_init__(self):
        for i, e in enumerate(self.run_order):
            if not 0 <= e.block < len(self.blocks):
                raise ConfigError("run_order", f"entry {i} names block {e.block} of {len(self.blocks)}")
            if e.before is not None and e.before.vector is not None:
                rows = dict(self.stream_vectors).get(e.before.vector)
                if rows is None or not 0 <= e.before.row < rows:
                    raise ConfigError("run_order", f"entry {i} adds row {e.before.row} of {e.before.vector!r}, "
                                                   "which the model does not declare")
            if e.cache_from is not None:
                if not 0 <= e.cache_from < i:
                    raise ConfigError("run_order", f"entry {i} reads the cache of entry {e.cache_from}, "
                                                   "which must come earlier")
                if self.run_order[e.cache_from].cache_from is not None:
                    raise ConfigError("run_order", f"entry {i} reads entry {e.cache_from}, "
                                                   "which has no cache of its own")
