"""Typed descriptions of the parts a decoder is assembled from.

A model is described by data only: a tuple of :class:`LayerSpec` (what each layer is made of), an
execution ``order`` (a list of layer indices, which may name a layer twice), and a few model-wide
sizes. Nothing in here knows an architecture's name; an architecture module turns its own
``config.json`` keys into these specs (see ``models/qwen3.py``).

Every spec is a frozen dataclass with a ``kind`` string. The part registries in
``parts/base.py`` map ``kind`` to the class that implements it, so a new kind of mixer,
feed-forward, norm or position encoding is added by registering a (spec, implementation) pair; no
spec in this file has to change for that.
"""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import Any


@dataclass(frozen=True)
class NormSpec:
    """Root-mean-square norm over the last ``dim`` elements: ``x * rsqrt(mean(x^2) + eps) * w``. With ``groups > 1``
    the elements are cut into that many equal consecutive parts, each divided by its own root mean square."""

    dim: int
    eps: float
    kind: str = "rmsnorm"
    groups: int = 1
    weight_offset: float = 0.0  # the stored weight lies this far below the one that multiplies (1.0: weights stored around zero)


@dataclass(frozen=True)
class RotarySpec:
    """Rotary position encoding over the first ``rotary_dim`` elements of each head.

    ``inv_freq[j] = theta ** (-2j / rotary_dim)``; pair ``j`` is ``(j, j + rotary_dim/2)`` with ``pairing ==
    "halves"`` and ``(2j, 2j + 1)`` with ``"neighbours"``. ``angles == "float64"``: the table of cosines and sines is
    worked out in double precision before it is rounded to float32 (``"float32"``: angles are float32 products).
    """

    rotary_dim: int
    theta: float
    kind: str = "rotary"
    pairing: str = "halves"
    angles: str = "float32"


@dataclass(frozen=True)
class YarnRotarySpec:
    """Rotary encoding over pairs of halves whose slow frequencies are stretched for contexts beyond the ``original`` one.

    With ``f_j = theta ** (-2j / rotary_dim)`` and ``dim(t) = rotary_dim * ln(original / (2 pi t)) / (2 ln theta)`` (the
    pair that makes ``t`` turns over the original context), ``lo = max(floor(dim(fast)), 0)``, ``hi = min(ceil(dim(slow)),
    rotary_dim - 1)``, ``ramp_j = clamp((j - lo) / max(hi - lo, 0.001), 0, 1)``: pair j turns at
    ``f_j / factor * ramp_j + f_j * (1 - ramp_j)``, and cosines and sines are multiplied by ``0.1 * ln(factor) + 1``. The
    table is worked out in double precision and rounded once.
    """

    rotary_dim: int
    theta: float
    factor: float
    original: float
    fast: float
    slow: float
    kind: str = "yarn_rotary"
    pairing: str = "halves"


@dataclass(frozen=True)
class ScaledRotarySpec:
    """Rotary encoding whose slow pairs are slowed for contexts beyond the ``original`` one. With ``f_j = theta ** (-2j / rotary_dim)``
    and the wavelength ``l_j = 2 pi / f_j``: pairs with ``l_j < original / high`` turn at ``f_j``, pairs with ``l_j > original / low``
    at ``f_j / factor``, and those between at ``(1 - s) f_j / factor + s f_j`` with ``s = (original / l_j - low) / (high - low)``.
    Cosines and sines are not multiplied by anything. The table is worked out in double precision and rounded once."""

    rotary_dim: int
    theta: float
    factor: float
    low: float
    high: float
    original: float
    kind: str = "scaled_rotary"
    pairing: str = "halves"


@dataclass(frozen=True)
class AttentionSpec:
    """Causal grouped-query attention over a paged key/value cache.

    ``window == 0`` means every earlier key is visible; ``window == w`` means a query at position
    ``p`` sees keys ``p-w+1 .. p``. ``qk_norm_eps`` is ``None`` when q and k are not normalised per
    head. ``position`` is ``None`` for a mixer without position encoding. ``cache_from`` names
    another layer (index into ``ModelPlan.layers``) whose keys and values this layer reads instead
    of writing its own.

    ``value_dim``: size of the value heads when it is not ``head_dim``. ``keep_first == f`` (with a window): keys
    ``0 .. f-1`` stay visible however far the window has moved. ``value_position``: a position encoding over the
    whole of ``value_dim`` that every value is turned by before it is cached, and every output turned back by at the
    query's position. ``names`` maps the roles ``q k v o q_norm k_norm`` to the checkpoint's suffixes.
    """

    hidden_size: int
    num_heads: int
    num_kv_heads: int
    head_dim: int
    scale: float
    qk_norm_eps: float | None = None
    window: int = 0
    position: Any | None = None
    cache_from: int | None = None
    kind: str = "attention"
    value_dim: int | None = None
    keep_first: int = 0
    value_position: Any | None = None
    names: tuple[tuple[str, str], ...] = ()
    # q and k are divided by their root mean square per head without a weight (with ``qk_norm_eps``)
    qk_norm_weight: bool = True
    # (coef, every) or None: the query at position p is multiplied by 1 + coef * ln(floor((p + 1) / every) + 1)
    query_temperature: tuple[float, int] | None = None
    # a projection to one number per head (role ``g`` of ``names``) whose sigmoid multiplies the head's output
    output_gate: bool = False
    # "head": q and k are normed head by head (a weight of ``head_dim``); "projection": over all rows of the projection at once,
    # before they are split into heads (weights of ``num_heads * head_dim`` and ``num_kv_heads * head_dim``)
    qk_norm_over: str = "head"
    # the values are the keys as projected, before the norm: there is no value projection (``value_dim`` is ``head_dim``)
    values_from_keys: bool = False
    # with a window: beside the window's keys a query sees one key and value for every block of ``pooled_block`` positions that
    # lies wholly before the window (block b: b P .. b P + P - 1, seen by position i when b P + P - 1 <= i - window): the mean of
    # the block's keys as the cache holds them and the mean of its values; tokens and blocks share one softmax. Tokens that have
    # left the window and whose block is not yet complete behind it are not seen
    pooled_block: int = 0
    # with q and k normed over the whole projection: > 0, a short causal convolution over time of that many taps on every channel of
    # q, k and v, directly behind the projections (``y_t = sum_j w[:, j] u_(t - taps + 1 + j)``, nothing but zeros ahead of a sequence's first token; weights
    # ``[channels, taps]`` under the roles ``q_conv k_conv v_conv``); the last ``taps - 1`` projections of a sequence are its state
    conv_taps: int = 0
    # > 0: every scaled score s becomes softcap * tanh(s / softcap) before the softmax
    softcap: float = 0.0
    # the softmax's denominator holds one more term, exp(0), that carries no value (a sink with the logit 0)
    unit_sink: bool = False

    @property
    def v_dim(self) -> int:
        return self.head_dim if self.value_dim is None else self.value_dim

    @property
    def kv_elements_per_token(self) -> int:
        """Key and value elements one token occupies in this layer's own pages (none when it reads another's)."""
        if self.cache_from is not None:
            return 0
        return self.num_kv_heads * (self.head_dim + self.v_dim) * (2 if self.pooled_block else 1)  # (the pooled blocks' pages)


@dataclass(frozen=True)
class LatentAttentionSpec:
    """Causal attention whose keys and values are linear maps of one latent per token.

    A token's projection gives ``latent_rank`` elements, RMS-normed with a weight: the latent c; and ``rotary_dim`` more, turned
    by the position: a key part that all heads share. Head h has the key ``[W_uk_h c | shared part]`` and the value
    ``W_uv_h c``; its query has ``head_dim`` elements that meet the first part and ``rotary_dim`` turned ones that meet the
    second. Only the latent and the shared part are cached. ``sink``: a learned logit per head that counts once in the
    softmax's denominator and has no value. ``output_gate`` as in :class:`AttentionSpec`. ``names`` maps the roles ``q dkv
    dkv_norm uk uv sink g o`` to the checkpoint's suffixes.
    """

    hidden_size: int
    num_heads: int
    head_dim: int
    rotary_dim: int
    value_dim: int
    latent_rank: int
    scale: float
    norm_eps: float
    position: Any
    sink: bool = False
    output_gate: bool = False
    names: tuple[tuple[str, str], ...] = ()
    kind: str = "latent_attention"
    # another layer (index into ``ModelPlan.layers``) whose latents and shared key parts this layer reads, as that layer's pages hold
    # them; it has no latent projection of its own (no ``dkv``, no ``dkv_norm``), but maps, queries and gates of its own
    cache_from: int | None = None

    @property
    def kv_elements_per_token(self) -> int:
        """Elements one token occupies in this layer's pages at most: the key ``[c | shared part]`` and its value rows (the
        latent once more; the whole key once more where the matrix-core kernels serve the layer)."""
        return 0 if self.cache_from is not None else 2 * (self.latent_rank + self.rotary_dim)


@dataclass(frozen=True)
class DecayStateSpec:
    """Linear attention with a fixed decay per head and a matrix of state per request and head:
    ``S_t = decay_h S_(t-1) + k_t v_t^T``, ``o_t = S_t^T q_t`` (no softmax, no denominator).

    ``input_activation`` ("none", "silu") is applied to the q, k and v projections; ``position`` (or None) turns the
    first elements of q and k; k is multiplied by ``key_scale``. ``output_norm``: "per_head" divides every head's
    output by its own root mean square (no weight); "all_heads" norms the concatenated heads together, with a weight.
    The normed outputs are multiplied by ``gate_activation`` ("silu", "sigmoid") of a fourth projection and go through
    the output projection. ``names`` maps the roles ``q k v g o norm`` to the checkpoint's suffixes.
    """

    hidden_size: int
    num_heads: int
    key_dim: int
    value_dim: int
    decay: tuple[float, ...]
    norm_eps: float
    input_activation: str = "none"
    position: Any | None = None
    key_scale: float = 1.0
    output_norm: str = "per_head"
    gate_activation: str = "silu"
    names: tuple[tuple[str, str], ...] = ()
    kind: str = "decay_state"

    @property
    def state_elements(self) -> int:
        return self.num_heads * self.key_dim * self.value_dim


@dataclass(frozen=True)
class DeltaRuleSpec:
    """Linear attention by the generalized delta rule, with a matrix of state per request and head (``head_dim x head_dim``,
    float32, zero at first). With r, k, v of ``num_heads x head_dim`` and the unit key ``u = k / sqrt(sum(k^2) + 1e-6)``::

        S_t = diag(w_t) S_(t-1) - (a_t * u_t) (u_t^T S_(t-1)) + k_t v_t^T,     o_t = S_t^T r_t

    (both terms read the old state). The decay per head and key channel is ``w = exp(-decay_coef * sigmoid(W_2 tanh(W_1 h) +
    w_0))`` with an inner size of ``decay_rank``; the removal rate ``a = sigmoid(W_a h + b_a)``. Each head's output is divided
    by its root mean square (``norm_eps``); the heads together are multiplied by a weight and by the sigmoid of a gate
    projection, and go through the output projection. ``names`` maps the roles ``r k v g a a_bias w1 w2 w0 norm o``."""

    hidden_size: int
    num_heads: int
    head_dim: int
    decay_rank: int
    norm_eps: float
    decay_coef: float = 0.6065306597126334  # exp(-1/2)
    names: tuple[tuple[str, str], ...] = ()
    kind: str = "delta_rule"

    @property
    def state_elements(self) -> int:
        return self.num_heads * self.head_dim * self.head_dim


@dataclass(frozen=True)
class TimeMixSpec:
    """Linear attention with a decay per token, head and key channel and a bonus for the current token, a ``head_dim x head_dim``
    float32 state per request and head (zero at first). With h' the input of the token before (zeros for a sequence's first), each of r,
    k, v, g, w reads its own blend ``h + (h' - h) * mu``; r, k, v are projections of theirs (``num_heads x head_dim``), ``gate =
    silu(W_g blend_g)``, the decay ``w = exp(-exp(W_2 tanh(W_1 blend_w) + w_0))`` (inner size ``decay_rank``), and::

        o_t = (S_(t-1) + diag(u) k_t v_t^T)^T r_t,        S_t = diag(w_t) S_(t-1) + k_t v_t^T

    Each head's o is divided by its root mean square (``norm_eps``); the heads together are multiplied by a weight and by the gate and go
    through the output projection. The last token's input is part of the state. ``names`` maps the roles ``mu_r mu_k mu_v mu_g mu_w r k
    v g w1 w2 w0 u norm o``."""

    hidden_size: int
    num_heads: int
    head_dim: int
    decay_rank: int
    norm_eps: float
    names: tuple[tuple[str, str], ...] = ()
    kind: str = "time_mix"

    @property
    def state_elements(self) -> int:
        return self.num_heads * self.head_dim * self.head_dim + self.hidden_size


@dataclass(frozen=True)
class PairMixerSpec:
    """Two mixers side by side that read the same input; the result is ``left_scale * left + right_scale * right``. Their tensors
    lie under ``<prefix>.<left_name>`` and ``<prefix>.<right_name>``; each keeps a cache or state of its own."""

    left: Any
    right: Any
    left_scale: float = 1.0
    right_scale: float = 1.0
    left_name: str = "left"
    right_name: str = "right"
    kind: str = "pair"

    @property
    def kv_elements_per_token(self) -> int:
        return sum(int(getattr(m, "kv_elements_per_token", 0)) for m in (self.left, self.right))


@dataclass(frozen=True)
class GatedMlpSpec:
    """Dense gated feed-forward: ``down(act(gate(x)) * up(x))`` without biases; ``activation`` is "silu" or
    "gelu_tanh"."""

    hidden_size: int
    intermediate_size: int
    activation: str = "silu"
    kind: str = "gated_mlp"
    names: tuple[tuple[str, str], ...] = ()  # roles ``gate up down`` -> the checkpoint's suffixes


@dataclass(frozen=True)
class ActivatedMlpSpec:
    """Dense feed-forward without a gate: ``down(act(up(x)))`` without biases; ``activation`` is "relu2" (the square of relu),
    "gelu_tanh" or "silu"."""

    hidden_size: int
    intermediate_size: int
    activation: str = "relu2"
    kind: str = "activated_mlp"
    names: tuple[tuple[str, str], ...] = ()  # roles ``up down`` -> the checkpoint's suffixes


@dataclass(frozen=True)
class TokenInputSpec:
    """An input that a layer takes from the token itself, behind its feed-forward: with e the elements ``[index * dim, (index + 1) *
    dim)`` of the token's row of the table ``table_name`` ``[vocab, *]``, ``y = W_proj (act(W_gate x) * e)`` and ``x += y / sqrt(mean(y^2) +
    eps) * w`` (an RMS norm with a plain weight). ``prefix`` names the tensors ``<prefix>.<gate|proj|norm>``."""

    table_name: str
    dim: int
    index: int
    eps: float
    prefix: str
    activation: str = "gelu_tanh"
    names: tuple[tuple[str, str], ...] = ()  # roles ``gate proj norm``


@dataclass(frozen=True)
class RoutedExpertsSpec:
    """A feed-forward of ``num_experts`` gated feed-forwards of ``intermediate_size`` each, of which a token uses the ``top_k``
    with the largest router logits (float32), weighted by the softmax over those logits alone. Tensors: ``<prefix>.<router>``
    ``[experts, hidden]`` and ``<prefix>.<expert><e>.<gate|up|down>``; ``names`` maps the roles ``router expert gate up down``."""

    hidden_size: int
    intermediate_size: int
    num_experts: int
    top_k: int
    activation: str = "silu"
    names: tuple[tuple[str, str], ...] = ()
    kind: str = "routed_experts"
    # what an activation with a limit clamps by ("clamped_sigmoid": g = min(gate, limit), u = clamp(up, -limit, limit),
    # g sigmoid(1.702 g) (u + 1))
    activation_limit: float = 0.0
    # "softmax_picked": the picks' weights are the softmax over the picked logits. "sigmoid_normalized": scores are sigmoid(z), the
    # picks are the largest scores among the experts of the ``keep_groups`` best of ``num_groups`` equal groups of neighbours (a
    # group's score: the sum of its two largest scores), and the weights are the picks' scores over their sum (+ 1e-20), times
    # ``route_scale``
    scoring: str = "softmax_picked"
    num_groups: int = 1
    keep_groups: int = 1
    route_scale: float = 1.0
    # > 0: one more expert of this size (``<prefix>.<shared>.<gate|up|down>``, the same form, ``shared_limit``) that every token
    # uses, multiplied by the sigmoid of one number per token (``<prefix>.<shared>.<shared_gate>`` ``[1, hidden]``)
    shared_size: int = 0
    shared_limit: float = 0.0
    # "softmax_all": scores are the softmax over all router outputs; the picks go by score + correction (a tensor under the role
    # ``correction``, when ``score_correction``), the weights are the picks' scores as they are, times ``route_scale``. The last
    # ``identity_experts`` router outputs (behind the ``num_experts`` with tensors) are identity experts: their result is the input
    identity_experts: int = 0
    score_correction: bool = False
    # False: an expert is ``down(act(up x))`` with an activation of :class:`ActivatedMlpSpec` (no gate rows)
    gated: bool = True
    # False: nothing multiplies the shared expert's result (no tensor under the role ``shared_gate``)
    shared_gated: bool = True


@dataclass(frozen=True)
class HyperConnectionSpec:
    """How a part of a layer is tied to ``streams`` residual streams: it reads ``sum_s in[s] x_s``, and once it has given y
    every stream is rewritten from the old ones, ``x_t = sum_s mix[s, t] x_s + out[t] y``. ``prefix`` names the tensors
    ``<prefix>.in [streams]``, ``<prefix>.out [streams]`` and ``<prefix>.mix [streams, streams]``."""

    streams: int
    prefix: str


@dataclass(frozen=True)
class LayerSpec:
    """One residual block: which mixer, which feed-forward, which norms, and how they are arranged.

    ``arrangement == "pre_norm"``: ``x += mixer(norm1(x)); x += ffn(norm2(x))``.
    ``arrangement == "parallel"``: ``h = norm1(x); x += residual_scale * (mixer(h) + ffn(h))``: one norm (``mixer_norm``)
    that both parts read; ``ffn`` may be None (then ``ffn_norm`` and its names are not used). With an ``ffn_norm`` the
    feed-forward has a norm of its own, of the same x: ``x += residual_scale * (mixer(norm1(x)) + ffn(norm2(x)))``.
    ``arrangement == "hyper_connections"``: as ``pre_norm`` over several residual streams: each part reads and rewrites them by
    its :class:`HyperConnectionSpec` (``mixer_streams``, ``ffn_streams``); ``ffn`` may be None.
    ``arrangement == "result_norm"``: the norms sit on the sublayers' results, and what a sublayer takes in is the stream as it stands:
    ``x += norm1(mixer(x)); x += norm2(ffn(x))``; ``ffn`` may be None. ``token_input`` (any arrangement that takes it): an input from
    the token itself behind the feed-forward (:class:`TokenInputSpec`).
    The ``*_prefix`` / ``*_name`` strings are the checkpoint names of this layer's tensors.
    """

    mixer: Any
    ffn: Any
    mixer_norm: Any
    ffn_norm: Any
    mixer_prefix: str
    ffn_prefix: str
    mixer_norm_name: str
    ffn_norm_name: str
    arrangement: str = "pre_norm"
    residual_scale: float = 1.0
    mixer_streams: Any | None = None
    ffn_streams: Any | None = None
    token_input: Any | None = None


@dataclass(frozen=True)
class ModelPlan:
    """Everything the generic decoder needs to build itself."""

    architecture: str
    vocab_size: int
    hidden_size: int
    layers: tuple[LayerSpec, ...]
    order: tuple[int, ...]
    final_norm: Any
    embed_name: str
    final_norm_name: str
    head_name: str
    tie_word_embeddings: bool
    max_position_embeddings: int
    eos_token_ids: tuple[int, ...] = field(default_factory=tuple)
    embedding_multiplier: float | None = None  # the looked-up rows are multiplied by it (None: as they are)
    logit_scale: float | None = None  # the logits are multiplied by it (None: as they are)
    residual_streams: int = 0  # > 0: that many residual streams, all the embedding at first, summed before the final norm
    token_table_columns: int = 0  # > 0: the row length of the table that the layers' token inputs read slices of

    def __post_init__(self) -> None:
        n = len(self.layers)
        if not self.order:
            raise ValueError("ModelPlan.order is empty")
        for i in self.order:
            if not 0 <= i < n:
                raise ValueError(f"ModelPlan.order names layer {i}, but there are {n} layers")
