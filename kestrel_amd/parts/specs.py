"""Parameters of the parts a model is put together from.

A specification is plain data: sizes and constants, nothing about the model it
ends up in. An architecture turns its ``config.json`` into a ``ModelPlan`` made of
these; the parts are then built from the plan through the registries of
``kestrel_amd.parts.base``. A specification of a kind that is not listed here (a
test's toy mixer, another feed-forward) is any object with a ``kind`` attribute
whose part class is registered under that kind.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, Mapping, Optional, Tuple


@dataclass(frozen=True)
class ParamSpec:
    """One tensor a part owns.

    ``role`` fixes how the tensor is held and initialised: ``matrix`` (2-D weight,
    model precision), ``vector`` (bias or gain), ``table`` (integer table, int32).
    ``init`` names the random-weights recipe: ``normal``, ``bias``, ``gain`` (around 1),
    ``shift`` (around 0) or ``fraction`` (around one half, inside 0 .. 1). An extent of -1 in ``shape`` leaves that
    size to the weights file (the part then reads it off the tensor it is bound to).
    """

    shape: Tuple[int, ...]
    role: str = "matrix"
    init: str = "normal"


@dataclass(frozen=True)
class NormSpec:
    """``offset``: what is added to the stored weight before it multiplies (1.0 for a weight stored around zero)."""

    kind: str
    dim: int
    eps: float
    bias: bool = True
    offset: float = 0.0


@dataclass(frozen=True)
class WavelengthScaling:
    """Rotary frequencies rescaled by wavelength ``l = 2 pi / f``: kept where ``l < original / high``, divided by
    ``factor`` where ``l > original / low``, and in between ``(1 - s) f / factor + s f`` with
    ``s = (original / l - low) / (high - low)``."""

    factor: float
    low: float
    high: float
    original: float


@dataclass(frozen=True)
class LinearScaling:
    """Rotary frequencies all divided by ``factor`` (positions stretched evenly)."""

    factor: float


@dataclass(frozen=True)
class PositionSpec:
    """Position encoding applied inside a mixer. ``kind`` ``none`` encodes nothing. ``pairing`` and ``scaling`` are
    read by the kind ``rotary`` (angles computed from frequencies, no table and so no longest sequence)."""

    kind: str
    rotary_dim: int = 0
    theta: float = 0.0
    max_positions: int = 0
    pairing: str = "halves"
    scaling: Optional[object] = None       # ``WavelengthScaling`` or ``LinearScaling``


@dataclass(frozen=True)
class LearnedPositionSpec:
    """One learned vector per position, added to the embedded tokens before the first block."""

    kind: str
    dim: int
    max_positions: int


@dataclass(frozen=True)
class ConcatLinearSpec:
    """A junction of the stack: the residual stream is replaced by one linear of the stream and the
    embedding output side by side, ``x <- W [x; x0]`` with ``W`` ``[dim, 2 dim]`` (the stream's columns first)."""

    kind: str
    dim: int


@dataclass(frozen=True)
class DistanceSlopes:
    """A bias on attention scores that grows with distance: the score of a query at place ``i`` against a key at
    place ``j`` is lowered by ``slope_h * (i - j)``, with ``slope_h = 2 ** (-exponent * (h + 1) / H)`` for query
    head ``h`` of ``H``."""

    exponent: float = 8.0

    def values(self, n_heads: int):
        return [2.0 ** (-self.exponent * (h + 1) / n_heads) for h in range(n_heads)]


@dataclass(frozen=True)
class QKNorm:
    """Queries and keys divided by a root mean square ``sqrt(mean(square) + eps)`` before rotation and scores: over
    every head by itself (``scope`` ``"head"``, gains of one head's size shared by all heads) or over the whole
    projection of a token (``"projection"``, gains of the projection's size). ``gain`` ``False``: no gains."""

    scope: str
    eps: float
    gain: bool = True


@dataclass(frozen=True)
class QueryGrowth:
    """Queries at place ``p`` multiplied by ``1 + coef * ln(floor((p + 1) / every) + 1)``."""

    coef: float
    every: int


@dataclass(frozen=True)
class DistanceBuckets:
    """A learned bias on attention scores by distance and head, ``rel[bucket(i - j), h]`` with ``rel`` ``[buckets, H]``:
    with ``half = buckets // 2``, ``bucket(n) = n`` for ``n < half``, else
    ``min(buckets - 1, half + floor(ln(n / half) / ln(far / half) * (buckets - half)))``. ``buckets`` ``None``: the
    number of rows of ``rel`` as stored says (``sized(rows)`` then gives the specification with the number in it)."""

    buckets: Optional[int]
    far: float

    def sized(self, buckets: int) -> "DistanceBuckets":
        return DistanceBuckets(int(buckets), self.far)

    def bucket(self, n: int) -> int:
        import math

        half = self.buckets // 2
        if n < half:
            return n
        return min(self.buckets - 1, half + int(math.floor(math.log(n / half) / math.log(self.far / half) * (self.buckets - half))))

    def distances(self) -> int:
        """Distances ``0 .. distances() - 1`` have buckets of their own to be looked up; every larger one falls into
        the last bucket, like ``distances() - 1`` does."""
        import math

        half = self.buckets // 2
        if self.buckets < 2 or not self.far > half:
            raise ValueError(f"distance buckets: {self.buckets} buckets need a far distance above {half}, got {self.far}")
        n = int(math.ceil(self.far))
        while n > 0 and self.bucket(n - 1) == self.buckets - 1:
            n -= 1
        return n + 1


@dataclass(frozen=True)
class ValueBlend:
    """Values of a layer blended with those another layer computed for the same token: the layer with ``role``
    ``"source"`` leaves its values for the step under ``name``; a layer with ``role`` ``"blend"`` replaces its own by
    ``(1 - w) v + w v_source`` with its learned scalar ``w`` before they are cached. (A source holds the scalar too
    and does not use it.)"""

    role: str
    name: str = "values"


@dataclass(frozen=True)
class CacheSpec:
    """What an attention mixer keeps per token: keys and values of ``n_kv_heads`` x ``head_dim``.

    ``window`` = number of most recent positions a query reads (``None``: all), which
    lets the cache manager give back pages that have fallen out of it. ``chunk`` = size of the chunks, counted
    from position 0, outside of which a query reads nothing (``None``: none): pages before the chunk of the next
    position go back as well.

    The cache manager asks a specification three things and nothing else, so a mixer that keeps
    something other than keys and values per token (one latent, another layout) brings a
    specification class of its own with the same three: ``window``; ``page_tensors(page_size)``,
    the tensors of one page by name with their shapes (the manager allocates each as
    ``[runs of layers, pages, *shape]`` and hands a layer its slice as ``LayerCache.tensors[name]``);
    and ``group_key``, equal for layers that can share a block table and a pool of pages.
    """

    n_kv_heads: int
    head_dim: int
    window: Optional[int] = None
    value_dim: Optional[int] = None     # size of a value head where it is not the keys' (``None``: ``head_dim``)
    chunk: Optional[int] = None
    # the first ``keep_first`` positions of a sequence stay readable after a window has passed them: their pages are
    # never given back while the request lives (``first_visible`` still names the window's start)
    keep_first: int = 0
    # value heads where they are fewer than key heads (several maps of keys over one head of values; ``None``: as many)
    value_heads: Optional[int] = None

    def first_visible(self, position: int) -> int:
        """The lowest key position that a query at ``position`` reads."""
        lo = 0
        if self.window is not None:
            lo = max(lo, position + 1 - self.window)
        if self.chunk is not None:
            lo = max(lo, position // self.chunk * self.chunk)
        return lo

    @property
    def bounded(self) -> bool:
        """Whether queries stop reading old keys at some point (pages can then be given back)."""
        return self.window is not None or self.chunk is not None

    def page_tensors(self, page_size: int) -> Dict[str, Tuple[int, ...]]:
        # values are kept transposed inside a page: eight consecutive keys of one channel are 16
        # bytes, which is what the MFMA attention kernels load at a time
        value_dim = self.head_dim if self.value_dim is None else self.value_dim
        value_heads = self.n_kv_heads if self.value_heads is None else self.value_heads
        return {"k": (self.n_kv_heads, page_size, self.head_dim), "v": (value_heads, value_dim, page_size)}

    @property
    def group_key(self) -> Tuple:
        value_dim = self.head_dim if self.value_dim is None else self.value_dim
        return ("kv", self.n_kv_heads, self.head_dim, self.window) + ((value_dim,) if value_dim != self.head_dim else ()) \
            + ((("chunk", self.chunk),) if self.chunk is not None else ()) \
            + ((("keep_first", self.keep_first),) if self.keep_first else ()) \
            + ((("value_heads", self.value_heads),) if self.value_heads is not None else ())


@dataclass(frozen=True)
class LatentCacheSpec:
    """What a latent attention mixer keeps per token: one row of ``latent_dim + shared_dim`` channels, the normalised
    key/value latent and the rotated key part that all heads share, side by side (the row is key and value at once)."""

    latent_dim: int
    shared_dim: int
    window: Optional[int] = None

    def page_tensors(self, page_size: int) -> Dict[str, Tuple[int, ...]]:
        return {"k": (1, page_size, self.latent_dim + self.shared_dim)}

    @property
    def group_key(self) -> Tuple:
        return ("latent", self.latent_dim, self.shared_dim, self.window)


@dataclass(frozen=True)
class StateSpec:
    """Per-request state of fixed size (one slot per live request), zeroed at admission."""

    shape: Tuple[int, ...]
    dtype: str = "float32"


@dataclass(frozen=True)
class AttentionSpec:
    kind: str
    dim: int
    n_heads: int
    n_kv_heads: int
    head_dim: int
    position: PositionSpec
    bias: bool = True
    scale: Optional[float] = None  # None: head_dim ** -0.5
    window: Optional[int] = None
    # size of a value head (``None``: ``head_dim``); the output projection then reads ``n_heads * value_dim`` columns
    value_dim: Optional[int] = None
    # the projections of queries, keys and values as three tensors (``q.weight``, ``k.weight``, ``v.weight``) instead of
    # one (``qkv.weight``); they are laid side by side when the weights are bound
    split_projections: bool = False
    # queries and keys divided, head by head, by their root mean square ``sqrt(mean(x^2) + eps)`` (no gain): its eps
    qk_unit_norm_eps: Optional[float] = None
    # scores lowered by a head's slope times the distance between query and key
    distance_slopes: Optional[DistanceSlopes] = None
    # one more term ``exp(sink)`` in the softmax's denominator that carries no value (``None``: none)
    sink: Optional[float] = None
    # a query reads only keys of its own chunk of this many positions (chunks counted from position 0)
    chunk: Optional[int] = None
    # queries and keys normalised, with learned gains, over a head or over the whole projection
    qk_norm: Optional[QKNorm] = None
    # a factor on the queries that grows with the place
    query_growth: Optional[QueryGrowth] = None
    # a learned bias per bucket of distance and head (tensor ``rel``)
    distance_buckets: Optional[DistanceBuckets] = None
    # values blended with those of another layer of the step (tensor ``vmix``)
    value_blend: Optional[ValueBlend] = None
    # the concatenated heads multiplied by ``sigmoid(gate.weight @ input)`` before the output projection
    output_gate: bool = False
    # the gate is one number per head (``gate.weight`` ``[n_heads, dim]``) instead of one per channel
    gate_per_head: bool = False
    # the values are the keys as projected, before any norm or rotation: there is no value projection
    # (``value_dim`` must be the head size)
    values_from_keys: bool = False
    # scores pass through ``softcap * tanh(score / softcap)`` after the scale
    softcap: Optional[float] = None
    # a learned score per head (tensor ``sinks`` ``[n_heads]``) for the valueless term of the softmax's denominator
    head_sinks: bool = False
    # the layer has no keys and values of its own: its schedule entry reads the cache of another (``reads_cache_of``),
    # and it holds no tensors of key and value projections or of their norm
    shares_kv: bool = False


@dataclass(frozen=True)
class WindowWithKeptFirst:
    """A query at place ``i`` reads the keys ``j <= i`` with ``i - j < size`` and, whatever their distance, the keys
    ``j < keep_first``; kept keys stand at their true places."""

    size: int
    keep_first: int = 0


@dataclass(frozen=True)
class DifferentialAttentionSpec:
    """Attention whose heads each hold two softmax maps over the same values, with queries ``[H, 2, head_dim]`` and keys
    ``[G, 2, head_dim]`` laid out head by head as ``[map 1, map 2]``, combined as ``a1 - lambda a2`` with
    ``lambda = exp(lq1 . lk1) - exp(lq2 . lk2) + lambda_init`` (one number for the layer), then divided by the root mean square
    over a head's values (``eps``, no gain) and multiplied by ``1 - lambda_init``. ``conv_taps``: a causal convolution over
    time on every channel of q, k and v right after their projections (``None``: none); ``mask`` ``None``: every ``j <= i``."""

    kind: str
    dim: int
    n_heads: int
    n_kv_heads: int
    head_dim: int
    value_dim: int
    scale: float
    lambda_init: float
    eps: float
    position: PositionSpec
    conv_taps: Optional[int] = None
    mask: Optional[WindowWithKeptFirst] = None


@dataclass(frozen=True)
class LatentAttentionSpec:
    """Attention whose queries, keys and values come from low-rank latents: ``c_q = rms(W_dq h) g_q`` (``q_rank``),
    ``q = W_uq c_q`` laid out per head as ``[head_dim plain, rot_dim rotated]``; ``W_dkv h`` gives the latent ``c`` (``kv_rank``,
    normalised with gains) and ``rot_dim`` channels of one rotated key part shared by all heads; a head's plain keys are
    ``W_uk c`` and its values ``W_uv c``. Every ``j <= i`` is seen. ``head_sinks``: one learned score per head that enters the
    softmax's denominator without a value. ``output_gate``: the heads times ``sigmoid(W_g h)`` before the output
    projection. ``position`` turns the ``rot_dim`` part."""

    kind: str
    dim: int
    n_heads: int
    head_dim: int
    rot_dim: int
    value_dim: int
    q_rank: int
    kv_rank: int
    scale: float
    eps: float
    position: PositionSpec
    head_sinks: bool = True
    output_gate: bool = True


@dataclass(frozen=True)
class ClampedGatedFeedForwardSpec:
    """``down(g sigmoid(slope g) (u + shift))`` with ``g = min(gate h, limit)`` and ``u = clamp(up h, -limit, limit)``."""

    kind: str
    dim: int
    hidden_dim: int
    limit: float
    slope: float = 1.702
    shift: float = 1.0
    activation: str = "none"
    bias: bool = False


@dataclass(frozen=True)
class PairEmbeddingSpec:
    """An embedding of token pairs added to the embedded tokens: row ``(prev * mul_prev + cur * mul_cur) mod buckets`` of a
    table of ``buckets + 1`` rows, and its last row for the first token of a sequence."""

    kind: str
    dim: int
    buckets: int
    mul_prev: int
    mul_cur: int
    vocab_size: int


@dataclass(frozen=True)
class PassVectorSpec:
    """A junction that adds a learned vector to the stream, one vector per passage (``[passages, dim]``;
    ``ScheduleEntry.passage`` says which)."""

    kind: str
    dim: int
    passages: int


@dataclass(frozen=True)
class DenseFeedForwardSpec:
    kind: str
    dim: int
    hidden_dim: int
    activation: str = "gelu_tanh"
    bias: bool = True


@dataclass(frozen=True)
class GatedFeedForwardSpec:
    """``down(act(gate h) * (up h))``."""

    kind: str
    dim: int
    hidden_dim: int
    activation: str = "gelu_tanh"
    bias: bool = False


@dataclass(frozen=True)
class RoutedExpertsSpec:
    """A mixture of gated feed-forwards ``down(act(gate h) * (up h))`` of which every token uses ``top``.

    The router has ``n_experts + n_identity`` outputs; its scores are their softmax (fp32). The choice goes by the scores
    plus a stored correction (tensor ``correction``), the weights by the scores alone: the chosen scores divided by
    their sum (+ 1e-20), times ``scale``. ``n_groups`` > 0: the router's outputs form that many equal groups of
    neighbours, a group counts by its largest choice score, and only outputs of the ``keep_groups`` best groups can be
    chosen. The last ``n_identity`` outputs are experts without tensors whose output is the input itself.
    ``shared_hidden``: a further expert of that hidden size that every token uses, times ``sigmoid(shared.sg h)`` (one
    number per token) if ``shared_gate``."""

    kind: str
    dim: int
    n_experts: int
    hidden_dim: int
    top: int
    scale: float = 1.0
    n_identity: int = 0
    n_groups: int = 0
    keep_groups: int = 0
    activation: str = "silu"
    shared_hidden: Optional[int] = None
    shared_gate: bool = True


@dataclass(frozen=True)
class DecayedMemorySpec:
    """A recurrent mixer in the manner of RWKV's time mixing: per head a state ``S`` ``[head_dim, head_dim]`` that decays
    channel by channel by a factor computed from the input (``parts/decayed_memory.py``). ``decay_rank``: the size of the
    low-rank bottleneck of the decay's projection (``None``: as the weights file has it)."""

    kind: str
    dim: int
    n_heads: int
    head_dim: int
    eps: float                      # of the norm of every head's read-out
    decay_rank: Optional[int] = None


@dataclass(frozen=True)
class MatrixMemorySpec:
    """A recurrent mixer whose state per head is a matrix ``[head_dim, value_dim]`` with a normaliser and a running
    maximum, written through exponential input and forget gates (``parts/matrix_memory.py``)."""

    kind: str
    dim: int
    n_heads: int
    head_dim: int
    value_dim: int
    gate_cap: float                 # gate pre-activations pass through ``cap * tanh(x / cap)``
    eps: float                      # of the norm of every head's read-out
    output_gate: bool = True


@dataclass(frozen=True)
class BranchesSpec:
    """Mixers side by side on the same input: the result is ``sum_i weights[i] * rms(branch_i(h)) * gain_i``, every
    branch's output normalised over the model width (``eps``) with a gain of its own."""

    kind: str
    dim: int
    branches: Tuple[object, ...]
    weights: Tuple[float, ...]
    eps: float


@dataclass(frozen=True)
class LayerSpec:
    """One block: its parts, how they are arranged, and where their tensors are named.

    ``arrangement``: ``parallel`` = ``x + mixer(norm(x)) + ff(norm(x))`` (one norm; ``feed_forward`` may be ``None``);
    ``sequential`` = ``x += mixer(norm(x)); x += ff(norm2(x))`` (``feed_forward`` and ``norm2`` may be ``None``: a mixer alone);
    ``parallel_two_norms`` = ``x + residual_scale * (mixer(norm(x)) + ff(norm2(x)))``, both norms of the same ``x``
    (``feed_forward`` and ``norm2`` may be ``None`` there: a layer of a mixer alone).
    ``output_norms`` = ``x += norm(mixer(x)); x += norm2(ff(x))``: the parts read the stream itself and the norms stand
    behind them (``feed_forward`` and ``norm2`` may be ``None``).
    ``names`` maps ``"<part>.<local tensor name>"`` (parts: ``norm``, ``norm2``, ``mixer``,
    ``feed_forward``) to the tensor's name in the checkpoint.
    """

    arrangement: str
    norm: object
    mixer: object
    feed_forward: object
    norm2: Optional[object] = None
    names: Mapping[str, str] = field(default_factory=dict)
    residual_scale: float = 1.0        # weight of the branches' sum in arrangements that have one


@dataclass(frozen=True)
class ScheduleEntry:
    """One run of a layer. ``reads_cache_of``: index of an earlier schedule entry whose
    cache this run reads instead of keeping one of its own. ``before``: name of a junction of the
    plan (``ModelPlan.junctions``) that the residual stream passes through right before this run; ``passage``: which
    passage through that junction this is (a junction whose tensors hold a row per passage reads it)."""

    layer: int
    reads_cache_of: Optional[int] = None
    before: Optional[str] = None
    passage: int = 0


@dataclass(frozen=True)
class ModelPlan:
    """Everything the generic decoder needs: parts layer by layer and their order."""

    architecture: str
    vocab_size: int
    dim: int
    max_positions: int
    layers: Tuple[LayerSpec, ...]
    schedule: Tuple[ScheduleEntry, ...]
    final_norm: object
    head_bias: bool
    tied_head: bool
    names: Mapping[str, str]  # "embedding", "final_norm.weight", "head.weight", ... -> tensor name
    eos_token_ids: Tuple[int, ...] = ()
    bos_token_id: Optional[int] = None
    # constants some architectures put around the stack (all neutral by default): a factor on the
    # looked-up embeddings, a factor on the logits, and a cap ``c`` that turns logits into c * tanh(logits / c)
    embedding_scale: float = 1.0
    logit_scale: float = 1.0
    logit_softcap: Optional[float] = None
    # a position encoding of the whole model (a specification whose part is registered as a position
    # encoding): its ``add_to_embeddings`` runs on the embedded tokens before the first block; its tensors
    # are named by ``names["position.<local name>"]``. ``None``: positions are the mixers' business.
    position: Optional[object] = None
    # junctions by name: specifications whose parts (registered as junctions) transform the residual stream between
    # runs of layers, where a schedule entry names one (``ScheduleEntry.before``); a junction named by several
    # entries runs with the same tensors each time; its tensors are named by ``names["junction.<name>.<local name>"]``
    junctions: Mapping[str, object] = field(default_factory=dict)
    # tensors of a checkpoint with these prefixes are passed over (parts that a configuration leaves out)
    ignored_prefixes: Tuple[str, ...] = ()

    def describe(self) -> Dict[str, object]:
        return {"architecture": self.architecture, "layers": len(self.layers), "schedule": len(self.schedule),
                "dim": self.dim, "vocab_size": self.vocab_size}
