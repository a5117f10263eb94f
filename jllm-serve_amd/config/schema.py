"""Typed description of a model: what config.json says, turned into per-layer specs.

The shapes follow the reference's records: ``Architecture.Core`` (model/Architecture.java:61-67),
``LayerSpec`` (model/LayerSpec.java:11-55), ``Attention.Gqa`` (model/Attention.java:48-115),
``Mlp.Dense`` (model/Mlp.java:7-22), ``RopeTable`` (model/RopeTable.java:20-52) and ``Scaling``
(model/Scaling.java:6-78). A family's switches are written into the per-layer specs, so nothing
below the parser ever looks at ``model_type`` (model/Architecture.java:17-20).

Every spec carries a ``kind`` string. The parts registry maps a kind to the class that runs it, so a
new mixer / feed-forward / norm / position encoding is a new spec class plus a registered part.
"""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any, Mapping, Optional, Sequence, Tuple


class ConfigError(ValueError):
    """A config.json that cannot be turned into a model (the reference's IllegalArgumentException)."""


# --------------------------------------------------------------------------- position encodings


@dataclass(frozen=True)
class RopeScaling:
    """Frequency rescaling of a rotary table (model/Scaling.java:6-78)."""

    kind: str = "none"  # none | linear | llama3 | yarn
    factor: float = 1.0
    original_max_positions: int = 0
    low_freq_factor: float = 1.0  # llama3
    high_freq_factor: float = 4.0  # llama3
    beta_fast: float = 32.0  # yarn
    beta_slow: float = 1.0  # yarn
    mscale: float = 1.0  # yarn
    mscale_all_dim: float = 0.0  # yarn
    attention_factor: float = 0.0  # yarn: 0 = derive from factor
    truncate: bool = True  # yarn


@dataclass(frozen=True)
class RopeSpec:
    """One rotary table (model/RopeTable.java:20-52). ``pairing`` "half" rotates (i, i + rotary_dim/2), "interleaved"
    rotates (2i, 2i + 1); the table is the same for both, the mixer's kernels apply it."""

    rotary_dim: int
    theta: float
    scaling: RopeScaling = RopeScaling()
    pairing: str = "half"
    kind: str = "rope"

    def __post_init__(self):
        # model/RopeTable.java:40-42
        if self.rotary_dim < 2 or self.rotary_dim % 2 != 0 or not (self.theta > 0):
            raise ConfigError(f"invalid rope table: rotary_dim={self.rotary_dim} theta={self.theta}")


@dataclass(frozen=True)
class LearnedPositionSpec:
    """A learned vector per position, added (unscaled) to the embedded rows at the input: row p of the tensor ``name``
    [``rows``, hidden]. It rotates nothing in the mixers."""

    name: str
    rows: int
    kind: str = "learned_position"


# --------------------------------------------------------------------------- norms


@dataclass(frozen=True)
class NormSpec:
    """RMSNorm with a plain gain (no 1+w) and the model's eps (model/Families.java:663, :793)."""

    eps: float
    kind: str = "rmsnorm"


@dataclass(frozen=True)
class LayerNormSpec:
    """Layer norm with a weight and a bias: (x - mean) / sqrt(mean of squared deviations + eps) * w + b. The bias is the
    tensor whose name is the weight's with ``bias_suffix`` added; ``bias`` False: the norm has a weight only."""

    eps: float
    bias_suffix: str = ".b"
    bias: bool = True
    kind: str = "layernorm"


@dataclass(frozen=True)
class DynTanhSpec:
    """Dynamic Tanh, a norm without statistics: tanh(alpha * x) * w + b element by element, with a scalar ``alpha`` and a
    vector ``b`` stored beside the weight under the weight's name with ``alpha_suffix`` / ``bias_suffix``. No mean, no
    variance, no eps."""

    bias_suffix: str = ".b"
    alpha_suffix: str = ".alpha"
    kind: str = "dyntanh"


# --------------------------------------------------------------------------- mixers


@dataclass(frozen=True)
class GqaNames:
    """Where the tensors of an attention layer are found in the checkpoint, relative to the layer's prefix and
    without the ``.weight`` / ``.bias`` ending (the reference keeps such a table per family as conversion rules,
    model/ModelConverter.java:38-49). ``qkv``: one tensor stacked [q | k | v] along the output rows, in place of
    the three."""

    q: str = "self_attn.q_proj"
    k: str = "self_attn.k_proj"
    v: str = "self_attn.v_proj"
    o: str = "self_attn.o_proj"
    q_norm: str = "self_attn.q_norm"
    k_norm: str = "self_attn.k_norm"
    qkv: Optional[str] = None


@dataclass(frozen=True)
class GqaSpec:
    """Grouped-query attention of one layer (model/Attention.java:48-115).

    ``window`` 0 means every earlier key is visible; otherwise the query at position p sees keys
    [max(0, p + 1 - window), p] (model/Attention.java:68-71). ``position`` indexes ModelConfig.positions
    (None = no position encoding). ``qk_norm``: per-head RMSNorm of q and k before the rotation with
    gains shared by all heads (model/Families.java:168).
    """

    heads: int
    kv_heads: int
    head_dim: int
    scale: float
    window: int = 0
    position: Optional[int] = 0
    qk_norm: bool = False
    qk_norm_eps: float = 1e-6
    bias: bool = False
    out_bias: bool = False
    names: GqaNames = GqaNames()
    kind: str = "gqa"

    @property
    def q_dim(self) -> int:
        return self.heads * self.head_dim

    @property
    def kv_dim(self) -> int:
        return self.kv_heads * self.head_dim

    @property
    def group(self) -> int:
        return self.heads // self.kv_heads


@dataclass(frozen=True)
class LatentAttentionNames:
    """Tensor names of a latent-attention mixer under the layer's prefix (no ending: the tensors are named bare)."""

    q: str = "mix.q"  # the query projection of a mixer without a query latent
    dq: str = "mix.dq"
    dq_norm: str = "mix.dq.norm"
    uq: str = "mix.uq"
    dkv: str = "mix.dkv"
    dkv_norm: str = "mix.dkv.norm"
    uk: str = "mix.uk"
    uv: str = "mix.uv"
    sink: str = "mix.sink"
    gate: str = "mix.g"
    o: str = "mix.o"
    ending: str = ""


@dataclass(frozen=True)
class LatentAttentionSpec:
    """Attention whose queries, keys and values pass through low-rank latents.

    Per position the layer caches the RMS-normed latent c (``kv_rank`` numbers) and one rotated key part of
    ``rot_dim`` numbers that all heads share; head h's unrotated key is W_uk[h] c and its value W_uv[h] c. A head's
    query has ``dim`` unrotated and ``rot_dim`` rotated entries and comes from a normed latent of ``q_rank``
    (``q_rank`` 0: straight from the input, by one projection ``q``).
    ``window`` 0 = all earlier keys, else the query at p sees keys p + 1 - window .. p. ``sink``: a learned number
    per head whose exponential joins the softmax's denominator. ``out_gate``: the concatenated heads are multiplied
    by sigmoid(W_g h) before the output product. ``owns_cache`` False: the run reads the cache of an earlier run (the
    schedule says which) and has no W_dkv. ``keep``: the window the cache must honour (the widest of the runs that
    read it; 0 = everything), which is what the cache manager sees."""

    heads: int
    dim: int
    rot_dim: int
    vdim: int
    q_rank: int
    kv_rank: int
    scale: float
    eps: float
    window: int = 0
    keep: int = 0
    position: Optional[int] = 0
    sink: bool = True
    out_gate: bool = True
    owns_cache: bool = True
    names: LatentAttentionNames = LatentAttentionNames()
    kind: str = "latent_attention"


@dataclass(frozen=True)
class WideAttentionNames:
    """Tensor names of an attention whose keys and values have sizes of their own, under the mixer's prefix; a bias is
    the weight's name with ``bias_suffix``, the gains of a norm over a whole projection the projection's name with
    ``norm_suffix``."""

    q: str = "q"
    k: str = "k"
    v: str = "v"
    gate: str = "g"
    o: str = "o"
    bias_suffix: str = ".b"
    norm_suffix: str = ".norm"
    lambda_q: Tuple[str, ...] = ("lq1", "lq2")  # differential attention: the vectors whose products give lambda
    lambda_k: Tuple[str, ...] = ("lk1", "lk2")
    sink: str = "sink"


@dataclass(frozen=True)
class WideAttentionSpec:
    """Causal grouped-query attention with a key size ``dim`` and a value size ``vdim`` of their own.

    ``maps`` 1: ordinary. ``maps`` 2 (differential attention): every query head and every key head holds two maps laid
    out [map 1 | map 2]; both are softmaxed alone over the same values and combined as a1 - lambda a2 with lambda =
    exp(lq1 . lk1) - exp(lq2 . lk2) + ``diff``; each head's result is divided by its root mean square (``eps``) and
    multiplied by 1 - ``diff``. ``qk_norm`` "whole": RMS norm with gains over the whole q projection and the whole k
    projection before the heads are split. ``position``: index of a rotary table (applied with its pairing on the
    first rotary_dim entries of every head) or None. ``softcap`` > 0: scores become softcap * tanh(score / softcap).
    ``q_temp_every`` > 0: q at position p is multiplied by 1 + q_temp_coef * ln(floor((p + 1) / q_temp_every) + 1).
    ``out_gate``: the concatenated heads are multiplied by sigmoid(W_g h) before the output product; ``gate_per_head``:
    W_g has one row per head and a head's whole output is multiplied by its one number. ``qk_norm`` "head": RMS norm of
    every q head and every k head alone, with one gain vector [dim] for all q heads and one for all k heads (the
    tensors ``<q>.norm`` / ``<k>.norm``). ``window`` > 0: the query at p sees keys p + 1 - window .. p, and, with
    ``keep_first``, also the keys at positions before ``keep_first`` (each still at the position it was written at). ``sink``: a
    learned number per head (tensor ``sink`` [heads]) whose exponential joins the softmax's denominator as it is: nothing
    is looked up for it, nothing is added to the weighted sum, and the scale does not touch it."""

    heads: int
    kv_heads: int
    dim: int
    vdim: int
    scale: float
    eps: float
    maps: int = 1
    diff: float = 0.0
    qk_norm: Optional[str] = None
    position: Optional[int] = None
    softcap: float = 0.0
    q_temp_coef: float = 0.0
    q_temp_every: int = 0
    bias: bool = True
    out_gate: bool = True
    window: int = 0
    keep_first: int = 0
    sink: bool = False
    gate_per_head: bool = False
    names: WideAttentionNames = WideAttentionNames()
    kind: str = "wide_attention"


@dataclass(frozen=True)
class GatedDeltaNames:
    """Tensor names of a gated-delta-rule mixer under its prefix; a projection's convolution taps are its name with
    ``conv_suffix``."""

    q: str = "q"
    k: str = "k"
    v: str = "v"
    beta: str = "b"
    decay: str = "a"
    a_log: str = "A_log"
    dt_bias: str = "dt_bias"
    norm: str = "norm"
    gate: str = "g"
    o: str = "o"
    conv_suffix: str = ".conv"
    # a decay or gate input that passes a narrow middle: W_up (W_down h)
    decay_down: str = "a1"
    decay_up: str = "a2"
    gate_down: str = "g1"
    gate_up: str = "g2"


@dataclass(frozen=True)
class GatedDeltaSpec:
    """A recurrent mixer: per head a matrix S [dim, vdim] that decays, is corrected towards the new value along the new
    key (the delta rule) and is read with the query. q and k have ``kv_heads`` heads of ``dim`` (value head h uses head
    h / (heads / kv_heads)), v has ``heads`` heads of ``vdim``; q, k and v pass a causal convolution of ``conv`` taps per
    channel and silu; q and k are made unit vectors (q also times dim^-1/2); the write strength is sigmoid(W_b h), the
    decay exp(-exp(A_log) softplus(W_a h + dt_bias)) per head; each head's read-out is divided by its root mean square
    (``eps``), multiplied by a gain shared by the heads and by silu(W_g h), and goes through W_o.

    ``decay`` "channel": one decay per head and key channel instead, g = exp(-exp(A_log_h) softplus(a + dt_bias)) with a
    and dt_bias laid out heads x dim, acting on the rows of S that belong to the key channels. ``decay_rank`` > 0: the
    decay's input is W_up (W_down h) through a middle of that many numbers (else one projection). ``gate_rank`` > 0: the
    same for the output gate's input. ``gate_fn``: "silu" or "sigmoid"."""

    heads: int
    kv_heads: int
    dim: int
    vdim: int
    conv: int
    eps: float
    names: GatedDeltaNames = GatedDeltaNames()
    decay: str = "head"
    decay_rank: int = 0
    gate_rank: int = 0
    gate_fn: str = "silu"
    kind: str = "gated_delta"


@dataclass(frozen=True)
class StateSpaceNames:
    """Tensor names of a state-space mixer under its prefix."""

    in_proj: str = "in"
    conv: str = "conv"
    conv_bias: str = "conv.b"
    dt_bias: str = "dt_bias"
    a_log: str = "A_log"
    skip: str = "D"
    norm: str = "norm"
    o: str = "o"


@dataclass(frozen=True)
class StateSpaceSpec:
    """A selective state-space mixer (the Mamba-2 form). One input projection gives [z | x | B | C | dt] with z and x
    of heads x ``vdim``, B and C of ``groups`` x ``state`` and one dt per head; x, B and C together pass a causal
    convolution of ``conv`` taps per channel with a bias, and silu. Per head (head h uses group h / (heads / groups)):
    dt = softplus(dt + dt_bias), S <- exp(-exp(A_log) dt) S + dt B x^T with S [state, vdim], y = S^T C + D x. The
    heads' y times silu(z) is RMS-normed in ``norm_groups`` equal parts (``eps``), multiplied by a weight, and goes
    through W_o."""

    heads: int
    vdim: int
    state: int
    groups: int
    norm_groups: int
    conv: int
    eps: float
    names: StateSpaceNames = StateSpaceNames()
    kind: str = "state_space"


@dataclass(frozen=True)
class ParallelMixerSpec:
    """Mixers side by side on the same input: the result is the sum of ``scales[i]`` times branch i's output. Branch
    i's tensors lie under the mixer's prefix + ``prefixes[i]``. At most one branch may own pages."""

    branches: Tuple[Any, ...]
    scales: Tuple[float, ...]
    prefixes: Tuple[str, ...]
    kind: str = "parallel"


# --------------------------------------------------------------------------- feed-forwards


@dataclass(frozen=True)
class GatedMlpNames:
    """Tensor names of a gated feed-forward under the layer's prefix, without ``.weight``. ``gate_up``: one tensor
    stacked [gate | up] along the output rows, in place of the two."""

    gate: str = "mlp.gate_proj"
    up: str = "mlp.up_proj"
    down: str = "mlp.down_proj"
    gate_up: Optional[str] = None
    ending: str = ".weight"  # what follows each name in the checkpoint ("" where tensors are named bare)


@dataclass(frozen=True)
class GatedMlpSpec:
    """Dense gated feed-forward: down(act(gate x) * up x) (model/Mlp.java:7-22). ``activation`` names the gate
    function of the product kernels: "silu", "gelu_tanh", or "swish_clamped" (g = min(gate, limit), u = clamp(up,
    -limit, limit), out = g * sigmoid(1.702 g) * (u + 1), with ``limit`` given here)."""

    hidden: int
    activation: str = "silu"
    names: GatedMlpNames = GatedMlpNames()
    limit: float = 0.0
    kind: str = "gated_mlp"


@dataclass(frozen=True)
class TableMoeNames:
    """Tensor names of a table-routed mixture of experts under the layer's prefix: expert e's tensors are
    ``<expert>{e}.<gate|up|down>``, the routing table ``table``, the shared expert's ``<shared>.<gate|up|down>``."""

    expert: str = "mlp.e"
    gate: str = "gate"
    up: str = "up"
    down: str = "down"
    table: str = "mlp.table"
    shared: str = "mlp.shared"
    ending: str = ""


@dataclass(frozen=True)
class TableMoeSpec:
    """A mixture of small gated feed-forwards without a router: an integer table [vocab, top] gives every token id
    its experts, each weighted 1 / top. Experts are "swish_clamped" gated feed-forwards of ``hidden`` with ``limit``;
    ``shared`` (a GatedMlpSpec or None) runs for every token and is added."""

    experts: int
    top: int
    hidden: int
    limit: float
    vocab: int
    shared: Any = None
    names: TableMoeNames = TableMoeNames()
    kind: str = "table_moe"


@dataclass(frozen=True)
class RoutedMoeNames:
    """Tensor names of a router-chosen mixture of experts under the layer's prefix: expert e's tensors are
    ``<expert>{e}.<gate|up|down>``, the router's weight ``router`` and the choice scores' correction ``correction``."""

    expert: str = "mlp.e"
    gate: str = "gate"
    up: str = "up"
    down: str = "down"
    router: str = "mlp.router"
    correction: str = "mlp.correction"
    shared_gate: str = "mlp.shared.sg"
    ending: str = ""


@dataclass(frozen=True)
class RoutedMoeSpec:
    """A mixture of small gated feed-forwards chosen by a router: scores s = sigmoid(W_router h) in fp32; the choice
    scores are s + correction (``correction`` False: s alone); the experts form ``groups`` equal groups of neighbours, a
    group's score is the sum of its two largest choice scores, and only experts of the ``keep`` best groups can be
    chosen; the ``top`` largest choice scores win; their weights are their s divided by the sum (+ 1e-20) times
    ``scale``. Experts are gated feed-forwards of ``hidden`` with the gate function ``activation`` (and its ``limit``
    where it has one). ``score`` "softmax": s = softmax(W_router h) over all experts. ``group_score`` "max": a group's
    score is its largest choice score. ``normalize`` False: the weights are the chosen s times ``scale``, not divided by
    their sum. ``shared`` (a GatedMlpSpec or None): a feed-forward that runs for every token and is added; with
    ``shared_gate`` it is first multiplied by sigmoid(W_sg h), one number per token (tensor ``shared_gate`` [1,
    hidden])."""

    experts: int
    top: int
    hidden: int
    scale: float = 1.0
    groups: int = 1
    keep: int = 1
    correction: bool = True
    activation: str = "silu"
    limit: float = 0.0
    score: str = "sigmoid"
    group_score: str = "top2"
    normalize: bool = True
    shared: Any = None
    shared_gate: bool = False
    names: RoutedMoeNames = RoutedMoeNames()
    kind: str = "routed_moe"


# --------------------------------------------------------------------------- layers and model


@dataclass(frozen=True)
class LayerSpec:
    """One decoder layer: which mixer, which feed-forward, which norms, and how they are arranged.

    ``arrangement`` "prenorm": x += mixer(norm(x)); x += ffn(norm(x)) (model/LayerSpec.java:18-19,
    cpu/CpuBackend.java:959-969). "parallel": with h = norm(x), x += mixer(h) + ffn(h): one norm, both sublayers read it.
    ``ffn`` None: the layer has no feed-forward (and no second norm). ``prefix`` is the tensor-name prefix of the layer's weights; the names under it
    are data of the specs (here the two norms', in the mixer's and feed-forward's specs theirs), so a checkpoint
    that names or stacks its tensors differently is a matter of the parser.
    """

    mixer: Any
    ffn: Any
    norm: Any
    prefix: str
    arrangement: str = "prenorm"
    norm_in_name: str = "input_layernorm"  # under the prefix, without the ending
    norm_post_name: str = "post_attention_layernorm"
    name_ending: str = ".weight"
    # arrangement "sandwich": x += norm_mixer_out(mixer(norm_in(x))); x += norm_ffn_out(ffn(norm_post(x)))
    norm_mixer_out_name: str = ""
    norm_ffn_out_name: str = ""
    mixer_prefix: str = ""  # under the layer's prefix, for mixers whose tensor names are relative to it
    # arrangement "hyper": the stream has ``streams`` copies per row; sublayer q reads u = sum_s in[s] x_s, and all
    # streams are rewritten at once, x_t <- sum_s mix[s, t] x_s + out[t] * sublayer(norm(u)), with the tensors
    # ``<prefix>.<hyper_names[q]>.in`` [streams], ``.out`` [streams], ``.mix`` [streams, streams] (row: the stream read, column: the stream written)
    streams: int = 1
    hyper_names: Tuple[str, str] = ("hc1", "hc2")


@dataclass(frozen=True)
class StreamVector:
    """A learned vector that is added to every row of the residual stream: row ``row`` of the tensor ``name``
    [``rows``, hidden]."""

    name: str
    rows: int
    row: int


@dataclass(frozen=True)
class StreamMix:
    """The stream is replaced by W [x; x0] right before a run: x the stream, x0 the embedding output of the same rows,
    W the tensor ``name`` [hidden, 2 hidden] with the stream's columns first."""

    name: str


@dataclass(frozen=True)
class ScheduleEntry:
    """One step of the layer schedule: run ``layer``; ``cache_from`` names an earlier schedule entry
    whose cache this run reads instead of writing one of its own (None = its own cache); ``add_before``: a vector
    that joins the stream right before this run (a layer that runs several times with one set of weights has a cache
    or state per run, and may be told which pass it is in this way); ``mix_before``: the stream is first mixed with the
    embedding output (before the vector joins)."""

    layer: int
    cache_from: Optional[int] = None
    add_before: Optional[StreamVector] = None
    mix_before: Optional[StreamMix] = None


@dataclass(frozen=True)
class ModelNames:
    """The checkpoint's names of the tensors outside the layers."""

    embed: str = "model.embed_tokens.weight"
    final_norm: str = "model.norm.weight"
    head: str = "lm_head.weight"
    embed_norm: str = ""  # the weight of a norm over the embedding output (ModelConfig.embed_norm)


@dataclass(frozen=True)
class ModelConfig:
    """The typed result of config.json (model/Architecture.java:61-67 plus model/Decoder.java:15-33)."""

    architecture: str
    model_type: str
    hidden: int
    vocab: int
    final_norm: Any
    layers: Tuple[LayerSpec, ...]
    positions: Tuple[Any, ...]
    schedule: Tuple[ScheduleEntry, ...]
    tie_embeddings: bool = False
    bos_token_id: int = -1
    eos_token_ids: Tuple[int, ...] = ()
    max_positions: int = 4096
    embed_scale: float = 1.0
    logit_scale: float = 1.0  # the logits are the head's product times this
    embed_norm: Any = None  # a norm spec: the embedded rows (with what the position encodings add) pass it first
    streams: int = 1  # residual streams per row: all start as the embedding output, the final norm reads their sum
    description: str = ""
    names: ModelNames = ModelNames()
    raw: Mapping[str, Any] = field(default_factory=dict, compare=False, repr=False)

    def __post_init__(self):
        n = len(self.layers)
        for i, e in enumerate(self.schedule):
            if not 0 <= e.layer < n:
                raise ConfigError(f"schedule entry {i} names layer {e.layer}, the model has {n}")
            if e.cache_from is not None and not 0 <= e.cache_from < i:
                raise ConfigError(f"schedule entry {i} reads the cache of entry {e.cache_from}, which does not run before it")

    @property
    def num_layers(self) -> int:
        return len(self.layers)


def default_schedule(n_layers: int) -> Tuple[ScheduleEntry, ...]:
    return tuple(ScheduleEntry(i) for i in range(n_layers))


def flatten(values: Sequence[Any]) -> str:
    return ",".join(str(v) for v in values)
