"""Small Gonurax configurations of the tests' own, model folders with seeded random weights for them, and the plain
implementation's logits for a set of requests."""

from __future__ import annotations

import torch

import plain_gonurax as plain


def attention(heads, kv_heads, dim, vdim, size, keep_first, rot_dims, base, scale, ff=None):
    return {"type": "attention",
            "mixer": {"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim, "scale": scale,
                      "mask": {"size": size, "keep_first": keep_first}, "rot": {"base": base, "dims": rot_dims}},
            "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def retention(heads, dim, vdim, decay, rot_dims, base, ff=None):
    return {"type": "retention",
            "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay), "rot": {"base": base, "dims": rot_dims}},
            "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def lightning(heads, dim, vdim, decay, ff=None):
    return {"type": "lightning", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay)},
            "mlp": None if ff is None else {"kind": "dense", "ff": ff}}


def model(vocab, width, groups, mult, eps, layers):
    return {"architecture": "Gonurax", "vocab": vocab, "width": width, "residual_mult": mult,
            "norm": {"eps": eps, "groups": groups}, "layers": layers}


def configs() -> dict[str, dict]:
    """Sizes, orders and constants that differ from one another in everything: windows shorter and longer than the
    prompts, no kept keys and several, as many key/value heads as heads and one, rotation over part of a head and over
    all of it, one norm group and several, a layer without feed-forward, a multiplier of 1, head sizes that are no
    power of two."""
    return {
        "P": model(300, 96, 3, 0.5, 1e-5, [
            retention(3, 32, 16, (0.9, 0.97, 0.995), 16, 1e4, ff=160),
            attention(4, 2, 32, 48, 24, 5, 16, 1e4, 0.2),
            lightning(2, 16, 24, (0.8, 0.99), ff=160),
            attention(4, 4, 16, 16, 40, 0, 16, 5e5, 0.25, ff=64)]),
        "Q": model(500, 128, 1, 1.0, 1e-6, [
            lightning(4, 48, 40, (0.5, 0.9, 0.99, 1.0), ff=192),
            attention(6, 1, 64, 32, 1000, 3, 32, 1e6, 0.11, ff=192),
            retention(2, 64, 96, (0.999, 0.98), 64, 5e4)]),
        "R": model(131, 80, 5, 0.8, 1e-6, [
            attention(3, 3, 24, 20, 17, 17, 24, 100.0, 0.3, ff=104),
            retention(5, 40, 12, (0.7, 0.9, 0.95, 0.99, 0.999), 20, 1e3, ff=104),
            lightning(1, 72, 136, (0.97,))]),
        # keys and values of one size that the matrix cores take: prompts in bfloat16 run the tiled attention kernel
        "S": model(210, 128, 2, 0.6, 1e-6, [
            attention(4, 2, 64, 64, 50, 6, 32, 1e4, 0.125, ff=128),
            lightning(2, 32, 32, (0.9, 0.99)),
            attention(8, 8, 32, 32, 100, 70, 32, 1e5, 0.2, ff=128)]),
        # sizes that are no multiple of 8 (products of this folder's kernels that take any size), five norm groups,
        # layers without a feed-forward
        "T": model(211, 100, 5, 0.9, 1e-4, [
            lightning(3, 12, 20, (0.9, 0.5, 0.99)),
            attention(5, 1, 20, 28, 9, 2, 10, 77.0, 0.4),
            retention(2, 36, 10, (0.95, 0.999), 36, 1e4, ff=52)]),
    }


BLOCK_SIZES = {"P": 16, "Q": 32, "R": 8, "S": 16, "T": 16}


def write_folder(folder: str, cfg: dict, seed: int = 0, std: float = 0.08) -> str:
    from mini_engine_amd.models.gonurax import GonuraxConfig, plan_from_config
    from mini_engine_amd.parts.decoder import Decoder
    from mini_engine_amd.weights import write_model_folder

    typed = GonuraxConfig.from_dict(cfg)
    wants = Decoder(plan_from_config(typed), torch.float32, "cpu").weight_wants()
    write_model_folder(folder, typed.to_config_json(), wants, seed=seed, dtype=torch.bfloat16, std=std, norm_std=0.1)
    return folder


def read_weights(folder: str) -> dict[str, torch.Tensor]:
    import os

    from safetensors.torch import load_file

    return {k: v.to(torch.float64) for k, v in load_file(os.path.join(folder, "model.safetensors")).items()}


def plain_logits(cfg: dict, weights: dict, requests: dict[str, list[int]]) -> dict[str, torch.Tensor]:
    return {rid: plain.forward(cfg, weights, toks)[0].to(torch.float32) for rid, toks in requests.items()}
