"""The Kifezen decoder: its ``config.json`` keys, and the plan that assembles it from parts.

A Kifezen model is a list of layers over ``streams`` residual streams (hyper-connections): a part reads a weighted sum of
the streams, is normed by an RMS norm whose weight is stored around zero (``1 + w`` multiplies), and its result rewrites all
streams at once by a mix matrix and an out vector of its own. The streams start as the embedding row and are summed before
the final norm; the head has its own table. Two mixers:

``attention``         grouped-query softmax attention without rotation: q and k divided by their root mean square per head
                      (no weight), the query multiplied by a temperature that grows with the logarithm of its position
                      in steps (``q_temp.coef``, ``q_temp.every``), the config's score scale, a sigmoid gate per head on the
                      output.
``latent_attention``  keys and values as linear maps of one normed latent per token (``kv_rank``) plus a rotated key part
                      that all heads share (``rot_dim``; rotation of halves with stretched slow frequencies,
                      ``rot.scaling``), a learned sink in the softmax's denominator, the same gate.

and two feed-forwards: ``dense`` (gated, silu) and ``moe`` (``router.experts`` gated experts of ``expert.ff``, ``router.top``
of them a token, weighted by the softmax over the picked router logits).

config.json keys: ``architecture``, ``vocab``, ``width``, ``streams``, ``norm.eps``, ``layers`` (each ``type``, ``mixer``, ``mlp``
or null). Tensor names: ``embed``, ``head``, ``final.norm``, ``l<i>.norm1``, ``l<i>.norm2``, ``l<i>.mix.*``, ``l<i>.mlp.*``
(``e<j>.gate|up|down``, ``router``), ``l<i>.hc1.*`` and ``l<i>.hc2.*`` (``in``, ``out``, ``mix``). A config without ``streams``
describes the same layers over one plain residual stream. A config gives no limit on the length of a sequence;
``max_position_embeddings`` here is the engine's own bound.
"""

from __future__ import annotations

import json
import os
from dataclasses import dataclass
from typing import Any

from ..config.registry import ArchitectureEntry, register_architecture
from ..config.specs import (
    AttentionSpec,
    GatedMlpSpec,
    HyperConnectionSpec,
    LatentAttentionSpec,
    LayerSpec,
    ModelPlan,
    NormSpec,
    RotarySpec,
    RoutedExpertsSpec,
    YarnRotarySpec,
)

ARCHITECTURE = "Kifezen"
MIXER_TYPES = ("attention", "latent_attention")
MLP_KINDS = ("dense", "moe")
MAX_POSITIONS = 1 << 20  # no key of the config bounds a sequence; the engine's max_model_len does

ATTENTION_NAMES = (("q", "q"), ("k", "k"), ("v", "v"), ("o", "o"), ("g", "g"))
LATENT_NAMES = (("q", "q"), ("dkv", "dkv"), ("dkv_norm", "dkv.norm"), ("uk", "uk"), ("uv", "uv"), ("sink", "sink"), ("g", "g"),
                ("o", "o"))
MLP_NAMES = (("gate", "gate"), ("up", "up"), ("down", "down"))
EXPERT_NAMES = (("router", "router"), ("expert", "e"), ("gate", "gate"), ("up", "up"), ("down", "down"))


def _need(d: dict, keys: tuple[str, ...], where: str) -> None:
    missing = [k for k in keys if k not in d]
    if missing:
        raise ValueError(f"{where} lacks required keys: {', '.join(missing)}")


@dataclass(frozen=True)
class KifezenConfig:
    """The numbers of ``config.json`` that the forward pass uses. ``layers`` keeps every layer's dictionary as it is written,
    checked for the keys its type needs. ``streams == 0``: the config names no streams (one plain residual stream)."""

    vocab: int
    width: int
    streams: int
    norm_eps: float
    layers: tuple[dict, ...]
    eos_token_ids: tuple[int, ...] = ()

    @classmethod
    def from_dict(cls, cfg: dict[str, Any], eos: Any = None) -> "KifezenConfig":
        _need(cfg, ("vocab", "width", "norm", "layers"), "config.json")
        _need(cfg["norm"], ("eps",), "config.json norm")
        streams = int(cfg.get("streams", 0) or 0)
        if streams < 0:
            raise ValueError(f"streams={streams} must not be negative")
        layers = []
        for i, layer in enumerate(cfg["layers"]):
            where = f"config.json layers[{i}]"
            _need(layer, ("type", "mixer"), where)
            kind, m = layer["type"], layer["mixer"]
            if kind not in MIXER_TYPES:
                raise ValueError(f"{where}: unknown mixer type {kind!r}; known: {', '.join(MIXER_TYPES)}")
            if kind == "attention":
                _need(m, ("heads", "kv_heads", "dim", "vdim", "scale"), where + ".mixer")
                if int(m["heads"]) % int(m["kv_heads"]):
                    raise ValueError(f"{where}: heads={m['heads']} is not a multiple of kv_heads={m['kv_heads']}")
                if m.get("q_temp") is not None:
                    _need(m["q_temp"], ("coef", "every"), where + ".mixer.q_temp")
                    if int(m["q_temp"]["every"]) < 1:
                        raise ValueError(f"{where}: q_temp.every must be positive")
            else:
                _need(m, ("heads", "dim", "rot_dim", "vdim", "kv_rank", "scale", "rot"), where + ".mixer")
                _need(m["rot"], ("base", "dims"), where + ".mixer.rot")
                if int(m["rot"]["dims"]) != int(m["rot_dim"]) or int(m["rot_dim"]) % 2 or int(m["rot_dim"]) < 2:
                    raise ValueError(f"{where}: rot.dims={m['rot']['dims']} must equal rot_dim={m['rot_dim']}, an even number")
                if m["rot"].get("scaling") is not None:
                    _need(m["rot"]["scaling"], ("factor", "original", "fast", "slow"), where + ".mixer.rot.scaling")
            mlp = layer.get("mlp")
            if mlp is not None:
                _need(mlp, ("kind",), where + ".mlp")
                if mlp["kind"] not in MLP_KINDS:
                    raise ValueError(f"{where}: unknown feed-forward kind {mlp['kind']!r}; known: {', '.join(MLP_KINDS)}")
                if mlp["kind"] == "dense":
                    _need(mlp, ("ff",), where + ".mlp")
                else:
                    _need(mlp, ("expert", "router"), where + ".mlp")
                    _need(mlp["expert"], ("ff",), where + ".mlp.expert")
                    _need(mlp["router"], ("experts", "top"), where + ".mlp.router")
                    if not 1 <= int(mlp["router"]["top"]) <= int(mlp["router"]["experts"]):
                        raise ValueError(f"{where}: router.top={mlp['router']['top']} of {mlp['router']['experts']} experts")
            layers.append(layer)
        if not layers:
            raise ValueError("config.json lists no layers")
        if eos is None:
            eos = cfg.get("eos_token_id")
        eos_ids = () if eos is None else ((int(eos),) if isinstance(eos, int) else tuple(int(e) for e in eos))
        return cls(vocab=int(cfg["vocab"]), width=int(cfg["width"]), streams=streams, norm_eps=float(cfg["norm"]["eps"]),
                   layers=tuple(layers), eos_token_ids=eos_ids)

    @classmethod
    def from_folder(cls, folder: str) -> "KifezenConfig":
        with open(os.path.join(folder, "config.json")) as f:
            return cls.from_dict(json.load(f))

    def to_config_json(self) -> dict[str, Any]:
        """A ``config.json`` dictionary that :meth:`from_dict` reads back to an equal object."""
        out = {"architecture": ARCHITECTURE, "vocab": self.vocab, "width": self.width, "norm": {"eps": self.norm_eps},
               "layers": [dict(layer) for layer in self.layers]}
        if self.streams:
            out["streams"] = self.streams
        return out


def position_spec(rot: dict):
    """The rotation of a latent attention layer: plain, or with its slow frequencies stretched (``rot.scaling``)."""
    sc = rot.get("scaling")
    if sc is None:
        return RotarySpec(rotary_dim=int(rot["dims"]), theta=float(rot["base"]), pairing="halves", angles="float64")
    return YarnRotarySpec(rotary_dim=int(rot["dims"]), theta=float(rot["base"]), factor=float(sc["factor"]),
                          original=float(sc["original"]), fast=float(sc["fast"]), slow=float(sc["slow"]))


def mixer_spec(cfg: KifezenConfig, kind: str, m: dict):
    if kind == "attention":
        temp = m.get("q_temp")
        return AttentionSpec(
            hidden_size=cfg.width, num_heads=int(m["heads"]), num_kv_heads=int(m["kv_heads"]), head_dim=int(m["dim"]),
            scale=float(m["scale"]), qk_norm_eps=cfg.norm_eps, qk_norm_weight=False, position=None, value_dim=int(m["vdim"]),
            query_temperature=None if temp is None else (float(temp["coef"]), int(temp["every"])), output_gate=True,
            names=ATTENTION_NAMES)
    return LatentAttentionSpec(
        hidden_size=cfg.width, num_heads=int(m["heads"]), head_dim=int(m["dim"]), rotary_dim=int(m["rot_dim"]),
        value_dim=int(m["vdim"]), latent_rank=int(m["kv_rank"]), scale=float(m["scale"]), norm_eps=cfg.norm_eps,
        position=position_spec(m["rot"]), sink=True, output_gate=True, names=LATENT_NAMES)


def ffn_spec(cfg: KifezenConfig, mlp: dict | None):
    if mlp is None:
        return None
    if mlp["kind"] == "dense":
        return GatedMlpSpec(hidden_size=cfg.width, intermediate_size=int(mlp["ff"]), activation="silu", names=MLP_NAMES)
    return RoutedExpertsSpec(hidden_size=cfg.width, intermediate_size=int(mlp["expert"]["ff"]),
                             num_experts=int(mlp["router"]["experts"]), top_k=int(mlp["router"]["top"]), activation="silu",
                             names=EXPERT_NAMES)


def plan_from_config(cfg: KifezenConfig) -> ModelPlan:
    norm = NormSpec(dim=cfg.width, eps=cfg.norm_eps, weight_offset=1.0)
    layers = []
    for i, layer in enumerate(cfg.layers):
        ffn = ffn_spec(cfg, layer.get("mlp"))
        if not cfg.streams and ffn is None:
            raise ValueError(f"config.json layers[{i}]: a layer without a feed-forward needs the streams' arrangement")
        layers.append(LayerSpec(
            mixer=mixer_spec(cfg, layer["type"], layer["mixer"]), ffn=ffn, mixer_norm=norm, ffn_norm=None if ffn is None else norm,
            mixer_prefix=f"l{i}.mix", ffn_prefix=f"l{i}.mlp", mixer_norm_name=f"l{i}.norm1", ffn_norm_name=f"l{i}.norm2",
            arrangement="hyper_connections" if cfg.streams else "pre_norm",
            mixer_streams=HyperConnectionSpec(cfg.streams, f"l{i}.hc1") if cfg.streams else None,
            ffn_streams=HyperConnectionSpec(cfg.streams, f"l{i}.hc2") if cfg.streams and ffn is not None else None))
    return ModelPlan(
        architecture=ARCHITECTURE, vocab_size=cfg.vocab, hidden_size=cfg.width, layers=tuple(layers),
        order=tuple(range(len(layers))), final_norm=norm, embed_name="embed", final_norm_name="final.norm",
        head_name="head", tie_word_embeddings=False, max_position_embeddings=MAX_POSITIONS, eos_token_ids=cfg.eos_token_ids,
        residual_streams=cfg.streams)


register_architecture(ArchitectureEntry(
    name=ARCHITECTURE, config_from_dict=KifezenConfig.from_dict, config_from_folder=KifezenConfig.from_folder,
    plan_from_config=plan_from_config))
