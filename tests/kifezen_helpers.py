"""Small Kifezen configurations of the tests' own, model folders with seeded random weights for them, and the plain
implementation's logits for a set of requests."""

from __future__ import annotations

import json
import os

import torch

import plain_kifezen as plain


def attention(heads, kv_heads, dim, vdim, scale, q_temp=None, mlp=None):
    m = {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale}
    if q_temp is not None:
        m["q_temp"] = {"coef": q_temp[0], "every": q_temp[1]}
    return {"type": "attention", "mixer": m, "mlp": mlp}


def latent(heads, dim, rot_dim, vdim, kv_rank, scale, base, scaling=None, mlp=None):
    rot = {"base": base, "dims": rot_dim}
    if scaling is not None:
        rot["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
    return {"type": "latent_attention",
            "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "kv_rank": kv_rank, "scale": scale, "rot": rot},
            "mlp": mlp}


def dense(ff):
    return {"kind": "dense", "ff": ff}


def moe(experts, top, ff):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


def model(vocab, width, streams, eps, layers):
    out = {"architecture": "Kifezen", "vocab": vocab, "width": width, "norm": {"eps": eps}, "layers": layers}
    if streams:
        out["streams"] = streams
    return out


def configs() -> dict[str, dict]:
    """Sizes, orders and constants that differ from one another in everything: one stream, three and four; as many key/value
    heads as heads and one; a temperature that steps every 7 positions, every 100, and none; rotation with and without
    stretched frequencies; one expert a token, all experts a token; a layer without a feed-forward; head sizes that are no
    multiple of 8; a latent wider than the heads it feeds."""
    return {
        "A": model(300, 96, 3, 1e-5, [
            attention(4, 2, 24, 16, 0.2, q_temp=(0.4, 7), mlp=moe(5, 2, 40)),
            latent(3, 16, 8, 24, 40, 0.17, 1e4, scaling=(4.0, 64, 16.0, 2.0), mlp=dense(136)),
            latent(2, 40, 16, 8, 24, 0.11, 500.0, mlp=moe(3, 3, 56))]),
        "B": model(500, 128, 1, 1e-6, [
            latent(4, 24, 40, 32, 56, 0.15, 3e4, scaling=(6.0, 256, 24.0, 1.0), mlp=moe(8, 1, 48)),
            attention(6, 6, 20, 20, 0.22, q_temp=(0.25, 100)),
            attention(2, 1, 64, 40, 0.09, mlp=dense(192))]),
        "C": model(131, 80, 4, 1e-6, [
            attention(5, 1, 12, 28, 0.3, q_temp=(1.5, 1), mlp=dense(104)),
            latent(5, 10, 6, 14, 18, 0.35, 77.0, scaling=(2.0, 20, 4.0, 0.5)),
            attention(4, 4, 16, 16, 0.25, q_temp=(0.1, 33), mlp=moe(16, 4, 24))]),
        # no streams named: the same layers over one plain residual stream
        "D": model(211, 64, 0, 1e-4, [
            latent(2, 16, 16, 16, 32, 0.2, 1e3, mlp=dense(72)),
            attention(4, 2, 16, 16, 0.25, q_temp=(0.3, 16), mlp=moe(4, 2, 32))]),
        # sizes that the matrix-core attention kernels take in bfloat16: keys and values of 64 elements; a latent key of
        # 96 + 32 elements under 16 heads
        "E": model(260, 128, 2, 1e-6, [
            attention(8, 2, 64, 64, 0.125, q_temp=(0.3, 40), mlp=dense(160)),
            latent(16, 24, 32, 16, 96, 0.13, 1e4, scaling=(4.0, 128, 16.0, 1.0), mlp=moe(6, 2, 64))]),
        # a latent wider than the model, whose cached key has more than 256 elements
        "F": model(150, 64, 2, 1e-6, [
            latent(2, 16, 16, 24, 272, 0.1, 1e4, mlp=dense(96)),
            attention(2, 2, 32, 32, 0.18, mlp=moe(4, 2, 32))]),
        # a cached key of 256 elements (the matrix-core kernels' largest head) under three streams; a key of 64 under one head
        "G": model(180, 64, 3, 1e-5, [
            latent(4, 16, 64, 16, 192, 0.08, 1e4, scaling=(16.0, 64, 8.0, 1.0), mlp=moe(3, 2, 40)),
            latent(1, 32, 16, 48, 48, 0.2, 2e3, mlp=dense(80))]),
        # head counts that are no power of two over keys that the matrix-core kernels take (64, 32 and 192 elements)
        "H": model(140, 96, 2, 1e-6, [
            latent(3, 24, 16, 8, 48, 0.15, 1e4, mlp=dense(64)),
            latent(5, 8, 8, 24, 24, 0.3, 300.0, scaling=(3.0, 32, 6.0, 1.0), mlp=moe(2, 1, 48)),
            latent(7, 16, 32, 16, 160, 0.07, 5e3, mlp=dense(64)),
            attention(6, 2, 32, 32, 0.2, q_temp=(0.2, 10))]),
        # sizes that are no multiple of 8 (a width of 100, feed-forwards of 52 and 20, a latent of 30 + 6): every product takes
        # the kernels that take any size; five streams: more than the product that norms the streams itself takes
        "I": model(211, 100, 5, 1e-5, [
            latent(3, 10, 6, 14, 30, 0.25, 1e3, scaling=(2.0, 16, 4.0, 1.0), mlp=moe(5, 2, 20)),
            attention(5, 1, 12, 20, 0.3, q_temp=(0.6, 3), mlp=dense(52))]),
    }


BLOCK_SIZES = {"A": 16, "B": 32, "C": 8, "D": 16, "E": 16, "F": 16, "G": 16, "H": 64, "I": 16}


def wants_of(cfg: dict):
    from mini_engine_amd.models.kifezen import KifezenConfig, plan_from_config
    from mini_engine_amd.parts.decoder import Decoder

    typed = KifezenConfig.from_dict(cfg)
    return typed, Decoder(plan_from_config(typed), torch.float32, "cpu").weight_wants()


def random_tensors(cfg: dict, seed: int, std: float = 0.08) -> dict[str, torch.Tensor]:
    """bfloat16 tensors by name: matrices from N(0, std); norm weights around zero (the latent's around one); stream
    coefficients around an even read, an identity mix and a unit write; sinks from N(0, 1); router rows wide apart, so
    that few picks are close calls."""
    _, wants = wants_of(cfg)
    g = torch.Generator().manual_seed(seed)
    s = int(cfg.get("streams", 0) or 0)
    out = {}
    for name, want in wants.items():
        x = torch.randn(want.shape, generator=g)
        if name.endswith(".dkv.norm"):
            t = 1.0 + 0.1 * x
        elif ".norm" in name:
            t = 0.1 * x
        elif name.endswith(".in"):
            t = 1.0 / s + 0.2 * x
        elif name.endswith(".out"):
            t = 1.0 + 0.2 * x
        elif name.endswith(".mix"):
            t = torch.eye(s) + 0.15 * x
        elif name.endswith(".sink"):
            t = x
        elif name.endswith(".router"):
            t = 0.6 * x
        else:
            t = std * x
        out[name] = t.to(torch.bfloat16)
    return out


def write_folder(folder: str, cfg: dict, seed: int = 0, tensors: dict | None = None) -> str:
    from mini_engine_amd.weights.safetensors_io import write_file

    typed, _ = wants_of(cfg)
    os.makedirs(folder, exist_ok=True)
    with open(os.path.join(folder, "config.json"), "w") as f:
        json.dump(typed.to_config_json(), f, indent=1)
    write_file(os.path.join(folder, "model.safetensors"), tensors if tensors is not None else random_tensors(cfg, seed), {"format": "pt"})
    return folder


def read_weights(folder: str) -> dict[str, torch.Tensor]:
    from safetensors.torch import load_file

    return {k: v.to(torch.float64) for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}


def plain_forward(cfg: dict, weights: dict, tokens: list[int], router_gaps: list | None = None, after_norm=None) -> torch.Tensor:
    """The plain implementation on a config that may name no streams: one stream that every part reads whole, keeps whole
    and adds its result to is the plain residual sum."""
    if not cfg.get("streams"):
        cfg = dict(cfg, streams=1)
        weights = dict(weights)
        for i, layer in enumerate(cfg["layers"]):
            for q in ("hc1", "hc2") if layer.get("mlp") is not None else ("hc1",):
                one = torch.ones(1, dtype=torch.float64)
                weights.update({f"l{i}.{q}.in": one, f"l{i}.{q}.out": one, f"l{i}.{q}.mix": one.view(1, 1)})
    return plain.forward(cfg, weights, tokens, router_gaps=router_gaps, after_norm=after_norm)


def rows_that_bear_rounding(cfg: dict, weights: dict, tokens: list[int], share: float = 0.015) -> torch.Tensor:
    """A mask of the positions whose plain logits move by less than ``share`` of the row's largest when every part's normed
    input is rounded to bfloat16. Random weights make some rows ill-conditioned (streams that nearly cancel in what a part
    reads, softmax weights on a knife's edge): there a bfloat16 engine and the plain implementation differ by what the
    model does to any rounding, not by a fault."""
    exact = plain_forward(cfg, weights, tokens)
    rounded = plain_forward(cfg, weights, tokens, after_norm=lambda z: z.to(torch.bfloat16).to(torch.float64))
    return (exact - rounded).abs().amax(-1) < share * exact.abs().amax(-1)


def rows_before_a_close_call(cfg: dict, weights: dict, tokens: list[int], share: float = 0.01) -> int:
    """How many leading positions of a sequence no router decides by less than ``share`` of its largest logit: up to there
    a rounding of the activations cannot change which experts a token uses (nor, through the keys and values that the
    token leaves, what later tokens read)."""
    gaps: list = []
    plain_forward(cfg, weights, tokens, gaps)
    if not gaps:
        return len(tokens)
    close = (torch.stack(gaps).amin(dim=0) < share).nonzero()
    return int(close[0]) if close.numel() else len(tokens)


def plain_logits(cfg: dict, weights: dict, requests: dict[str, list[int]]) -> dict[str, torch.Tensor]:
    return {rid: plain_forward(cfg, weights, toks).to(torch.float32) for rid, toks in requests.items()}
