"""The Gonurax decoder: its ``config.json`` keys, and the plan that assembles it from parts.

A Gonurax model is a list of layers, each with one of three mixers and an optional dense feed-forward, arranged in
parallel: ``h = norm(x); x += residual_mult * (mixer(h) + ff(h))``, with a root-mean-square norm in groups. The head is
the embedding table. The three mixers:

``attention``  grouped-query softmax attention with a per-head q/k norm (one weight for all heads), rotation of
               neighbouring pairs over the first ``rot.dims`` elements, values turned by their own position over all of
               their elements (and outputs turned back), the config's score scale, and a sliding window that keeps the
               first tokens (``mask.size``, ``mask.keep_first``).
``retention``  linear attention with a decay per head: rotation of halves on q and k, k times ``dim ** -0.5``, every
               head's output over its own root mean square, a silu gate.
``lightning``  linear attention with a decay per head: silu on q, k and v, all heads normed together with a weight, a
               sigmoid gate.

config.json keys: ``architecture``, ``vocab``, ``width``, ``residual_mult``, ``norm`` (``eps``, ``groups``), ``layers``
(each ``type``, ``mixer`` with the mixer's sizes, ``mlp`` with ``kind`` and ``ff``, or null). Tensor names:
``embed``, ``final.norm``, ``l<i>.norm1``, ``l<i>.mix.{q,k,v,g,o,norm,q.norm,k.norm}``, ``l<i>.mlp.{gate,up,down}``.
A config gives no limit on the length of a sequence; ``max_position_embeddings`` here is the engine's own bound.
"""

from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import Any

from ..config.registry import ArchitectureEntry, register_architecture
from ..config.specs import AttentionSpec, DecayStateSpec, GatedMlpSpec, LayerSpec, ModelPlan, NormSpec, RotarySpec

ARCHITECTURE = "Gonurax"
MIXER_TYPES = ("attention", "retention", "lightning")
MAX_POSITIONS = 1 << 20  # no key of the config bounds a sequence; the engine's max_model_len does

ATTENTION_NAMES = (("q", "q"), ("k", "k"), ("v", "v"), ("o", "o"), ("q_norm", "q.norm"), ("k_norm", "k.norm"))
STATE_NAMES = (("q", "q"), ("k", "k"), ("v", "v"), ("g", "g"), ("o", "o"), ("norm", "norm"))
MLP_NAMES = (("gate", "gate"), ("up", "up"), ("down", "down"))


def _need(d: dict, keys: tuple[str, ...], where: str) -> None:
    missing = [k for k in keys if k not in d]
    if missing:
        raise ValueError(f"{where} lacks required keys: {', '.join(missing)}")


@dataclass(frozen=True)
class GonuraxConfig:
    """The numbers of ``config.json`` that the forward pass uses. ``layers`` keeps every layer's dictionary as it is
    written (type, mixer sizes, feed-forward), checked for the keys its type needs."""

    vocab: int
    width: int
    residual_mult: float
    norm_eps: float
    norm_groups: int
    layers: tuple[dict, ...]
    eos_token_ids: tuple[int, ...] = ()

    @classmethod
    def from_dict(cls, cfg: dict[str, Any], eos: Any = None) -> "GonuraxConfig":
        _need(cfg, ("vocab", "width", "residual_mult", "norm", "layers"), "config.json")
        _need(cfg["norm"], ("eps", "groups"), "config.json norm")
        width, groups = int(cfg["width"]), int(cfg["norm"]["groups"])
        if groups < 1 or width % groups:
            raise ValueError(f"width={width} cannot be cut into norm.groups={groups} equal parts")
        layers = []
        for i, layer in enumerate(cfg["layers"]):
            where = f"config.json layers[{i}]"
            _need(layer, ("type", "mixer"), where)
            kind, m = layer["type"], layer["mixer"]
            if kind not in MIXER_TYPES:
                raise ValueError(f"{where}: unknown mixer type {kind!r}; known: {', '.join(MIXER_TYPES)}")
            if kind == "attention":
                _need(m, ("heads", "kv_heads", "dim", "vdim", "rot", "scale", "mask"), where + ".mixer")
                _need(m["rot"], ("base", "dims"), where + ".mixer.rot")
                _need(m["mask"], ("size", "keep_first"), where + ".mixer.mask")
                if int(m["heads"]) % int(m["kv_heads"]):
                    raise ValueError(f"{where}: heads={m['heads']} is not a multiple of kv_heads={m['kv_heads']}")
                if int(m["vdim"]) % 2:
                    raise ValueError(f"{where}: vdim={m['vdim']} must be even: the values are turned in pairs")
                if int(m["mask"]["size"]) < 1 or int(m["mask"]["keep_first"]) < 0:
                    raise ValueError(f"{where}: mask.size must be positive and mask.keep_first not negative")
            else:
                _need(m, ("heads", "dim", "vdim", "decay"), where + ".mixer")
                if len(m["decay"]) != int(m["heads"]):
                    raise ValueError(f"{where}: {len(m['decay'])} decays for {m['heads']} heads")
                if kind == "retention":
                    _need(m, ("rot",), where + ".mixer")
                    _need(m["rot"], ("base", "dims"), where + ".mixer.rot")
            if "rot" in m and (int(m["rot"]["dims"]) % 2 or not 0 < int(m["rot"]["dims"]) <= int(m["dim"])):
                raise ValueError(f"{where}: rot.dims={m['rot']['dims']} must be even and at most dim={m['dim']}")
            mlp = layer.get("mlp")
            if mlp is not None:
                _need(mlp, ("kind", "ff"), where + ".mlp")
                if mlp["kind"] != "dense":
                    raise ValueError(f"{where}: unknown feed-forward kind {mlp['kind']!r}; known: dense")
            layers.append(layer)
        if not layers:
            raise ValueError("config.json lists no layers")
        if eos is None:
            eos = cfg.get("eos_token_id")
        eos_ids = () if eos is None else ((int(eos),) if isinstance(eos, int) else tuple(int(e) for e in eos))
        return cls(vocab=int(cfg["vocab"]), width=width, residual_mult=float(cfg["residual_mult"]),
                   norm_eps=float(cfg["norm"]["eps"]), norm_groups=groups, layers=tuple(layers), eos_token_ids=eos_ids)

    @classmethod
    def from_folder(cls, folder: str) -> "GonuraxConfig":
        with open(os.path.join(folder, "config.json")) as f:
            return cls.from_dict(json.load(f))

    def to_config_json(self) -> dict[str, Any]:
        """A ``config.json`` dictionary that :meth:`from_dict` reads back to an equal object."""
        return {"architecture": ARCHITECTURE, "vocab": self.vocab, "width": self.width, "residual_mult": self.residual_mult,
                "norm": {"eps": self.norm_eps, "groups": self.norm_groups}, "layers": [dict(layer) for layer in self.layers]}


def mixer_spec(cfg: GonuraxConfig, kind: str, m: dict):
    heads, d, dv = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    if kind == "attention":
        rot = m["rot"]
        return AttentionSpec(
            hidden_size=cfg.width, num_heads=heads, num_kv_heads=int(m["kv_heads"]), head_dim=d, scale=float(m["scale"]),
            qk_norm_eps=cfg.norm_eps, window=int(m["mask"]["size"]), keep_first=int(m["mask"]["keep_first"]), value_dim=dv,
            position=RotarySpec(rotary_dim=int(rot["dims"]), theta=float(rot["base"]), pairing="neighbours", angles="float64"),
            value_position=RotarySpec(rotary_dim=dv, theta=float(rot["base"]), pairing="neighbours", angles="float64"),
            names=ATTENTION_NAMES)
    decay = tuple(float(v) for v in m["decay"])
    if kind == "retention":
        rot = m["rot"]
        return DecayStateSpec(
            hidden_size=cfg.width, num_heads=heads, key_dim=d, value_dim=dv, decay=decay, norm_eps=cfg.norm_eps,
            input_activation="none", key_scale=d ** -0.5, output_norm="per_head", gate_activation="silu",
            position=RotarySpec(rotary_dim=int(rot["dims"]), theta=float(rot["base"]), pairing="halves", angles="float64"),
            names=STATE_NAMES)
    return DecayStateSpec(
        hidden_size=cfg.width, num_heads=heads, key_dim=d, value_dim=dv, decay=decay, norm_eps=cfg.norm_eps,
        input_activation="silu", key_scale=1.0, output_norm="all_heads", gate_activation="sigmoid", position=None,
        names=STATE_NAMES)


def plan_from_config(cfg: GonuraxConfig) -> ModelPlan:
    norm = NormSpec(dim=cfg.width, eps=cfg.norm_eps, groups=cfg.norm_groups)
    layers = []
    for i, layer in enumerate(cfg.layers):
        mlp = layer.get("mlp")
        ffn = None if mlp is None else GatedMlpSpec(hidden_size=cfg.width, intermediate_size=int(mlp["ff"]),
                                                    activation="gelu_tanh", names=MLP_NAMES)
        layers.append(LayerSpec(
            mixer=mixer_spec(cfg, layer["type"], layer["mixer"]), ffn=ffn, mixer_norm=norm, ffn_norm=None,
            mixer_prefix=f"l{i}.mix", ffn_prefix=f"l{i}.mlp", mixer_norm_name=f"l{i}.norm1", ffn_norm_name="",
            arrangement="parallel", residual_scale=cfg.residual_mult))
    return ModelPlan(
        architecture=ARCHITECTURE, vocab_size=cfg.vocab, hidden_size=cfg.width, layers=tuple(layers),
        order=tuple(range(len(layers))), final_norm=norm, embed_name="embed", final_norm_name="final.norm",
        head_name="head", tie_word_embeddings=True, max_position_embeddings=MAX_POSITIONS, eos_token_ids=cfg.eos_token_ids)


register_architecture(ArchitectureEntry(
    name=ARCHITECTURE, config_from_dict=GonuraxConfig.from_dict, config_from_folder=GonuraxConfig.from_folder,
    plan_from_config=plan_from_config))
