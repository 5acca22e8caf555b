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

    @property
    def v_dim(self) -> int:
        return self.head_dim if self.value_dim is None else self.value_dim

    @property
    def kv_elements_per_token(self) -> int:
        """Key and value elements one token occupies in this layer's own pages (none when it reads another's)."""
        return 0 if self.cache_from is not None else self.num_kv_heads * (self.head_dim + self.v_dim)


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
class GatedMlpSpec:
    """Dense gated feed-forward: ``down(act(gate(x)) * up(x))`` without biases; ``activation`` is "silu" or
    "gelu_tanh"."""

    hidden_size: int
    intermediate_size: int
    activation: str = "silu"
    kind: str = "gated_mlp"
    names: tuple[tuple[str, str], ...] = ()  # roles ``gate up down`` -> the checkpoint's suffixes


@dataclass(frozen=True)
class LayerSpec:
    """One residual block: which mixer, which feed-forward, which norms, and how they are arranged.

    ``arrangement == "pre_norm"``: ``x += mixer(norm1(x)); x += ffn(norm2(x))``.
    ``arrangement == "parallel"``: ``h = norm1(x); x += residual_scale * (mixer(h) + ffn(h))``: one norm (``mixer_norm``)
    that both parts read; ``ffn`` may be None (then ``ffn_norm`` and its names are not used).
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

    def __post_init__(self) -> None:
        n = len(self.layers)
        if not self.order:
            raise ValueError("ModelPlan.order is empty")
        for i in self.order:
            if not 0 <= i < n:
                raise ValueError(f"ModelPlan.order names layer {i}, but there are {n} layers")
