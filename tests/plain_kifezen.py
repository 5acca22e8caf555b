"""A plain, slow implementation of the Kifezen design in double precision: one function per mechanism, whole
sequences at once, no cache. It shares no code with the package; the tests compare the engine against it.

A model is ``(cfg, w)``: the ``config.json`` dictionary and a dictionary of float64 tensors by checkpoint name.
"""

from __future__ import annotations

import math

import torch

F = torch.float64


def rms_unit(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x over its root mean square along the last axis (eps inside the root)."""
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def offset_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    """RMS norm whose stored weight lies around zero."""
    return rms_unit(x, eps) * (1.0 + w)


def plain_norm(x: torch.Tensor, w: torch.Tensor, eps: float) -> torch.Tensor:
    return rms_unit(x, eps) * w


def streams_read(streams: torch.Tensor, w_in: torch.Tensor) -> torch.Tensor:
    """streams [S, T, W] -> the sublayer's input [T, W]."""
    return torch.einsum("s,stw->tw", w_in, streams)


def streams_write(streams: torch.Tensor, y: torch.Tensor, w_mix: torch.Tensor, w_out: torch.Tensor) -> torch.Tensor:
    """new[t] = sum_s mix[s, t] old[s] + out[t] y, all streams from the old ones."""
    return torch.einsum("sk,stw->ktw", w_mix, streams) + w_out[:, None, None] * y[None]


def query_temperature(positions: torch.Tensor, coef: float, every: int) -> torch.Tensor:
    return 1.0 + coef * torch.log(torch.floor((positions + 1) / every) + 1.0)


def causal_softmax(scores: torch.Tensor, sink: torch.Tensor | None = None) -> torch.Tensor:
    """scores [H, T, T]; key j is visible to query i when j <= i. ``sink`` [H]: one more term exp(sink) in every
    denominator, with no value."""
    t = scores.shape[-1]
    mask = torch.ones(t, t, dtype=torch.bool).tril()
    scores = scores.masked_fill(~mask, -math.inf)
    if sink is None:
        return torch.softmax(scores, dim=-1)
    m = torch.maximum(scores.max(dim=-1, keepdim=True).values, sink[:, None, None])
    e = torch.exp(scores - m)
    return e / (e.sum(dim=-1, keepdim=True) + torch.exp(sink[:, None, None] - m))


def softmax_attention(h: torch.Tensor, m: dict, w: dict, pre: str, eps: float) -> torch.Tensor:
    """Grouped-query attention without rotation: unit-norm q and k per head, a temperature on q by position, a gate per
    head on the output."""
    t = h.shape[0]
    nh, nkv, d, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q = (h @ w[pre + ".q"].T).view(t, nh, d)
    k = (h @ w[pre + ".k"].T).view(t, nkv, d)
    v = (h @ w[pre + ".v"].T).view(t, nkv, dv)
    q, k = rms_unit(q, eps), rms_unit(k, eps)
    pos = torch.arange(t, dtype=F)
    if m.get("q_temp") is not None:
        q = q * query_temperature(pos, float(m["q_temp"]["coef"]), int(m["q_temp"]["every"]))[:, None, None]
    rep = nh // nkv
    k = k.repeat_interleave(rep, dim=1)
    v = v.repeat_interleave(rep, dim=1)
    p = causal_softmax(torch.einsum("ihd,jhd->hij", q, k) * float(m["scale"]))
    o = torch.einsum("hij,jhd->ihd", p, v)
    gate = torch.sigmoid(h @ w[pre + ".g"].T)  # [T, H]
    return (o * gate[:, :, None]).reshape(t, nh * dv) @ w[pre + ".o"].T


def yarn_frequencies(rot: dict) -> tuple[torch.Tensor, float]:
    """(frequency per pair [dims/2], what cosines and sines are multiplied by)."""
    dims, base = int(rot["dims"]), float(rot["base"])
    i = torch.arange(dims // 2, dtype=F)
    f = base ** (-2.0 * i / dims)
    sc = rot.get("scaling")
    if not sc:
        return f, 1.0
    factor, original = float(sc["factor"]), float(sc["original"])

    def dim_of(turns: float) -> float:
        return dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

    lo = max(math.floor(dim_of(float(sc["fast"]))), 0)
    hi = min(math.ceil(dim_of(float(sc["slow"]))), dims - 1)
    ramp = ((i - lo) / max(hi - lo, 0.001)).clamp(0.0, 1.0)
    return f / factor * ramp + f * (1.0 - ramp), 0.1 * math.log(factor) + 1.0


def rotate_halves(x: torch.Tensor, positions: torch.Tensor, rot: dict) -> torch.Tensor:
    """x [T, ..., n]: the first rot.dims elements turned, element i with element i + dims/2."""
    dims = int(rot["dims"])
    f, mult = yarn_frequencies(rot)
    ang = positions[:, None] * f[None, :]
    shape = (x.shape[0],) + (1,) * (x.dim() - 2) + (dims // 2,)
    c, s = (torch.cos(ang) * mult).view(shape), (torch.sin(ang) * mult).view(shape)
    u, v = x[..., :dims // 2], x[..., dims // 2:dims]
    return torch.cat((u * c - v * s, v * c + u * s, x[..., dims:]), dim=-1)


def latent_attention(h: torch.Tensor, m: dict, w: dict, pre: str, eps: float) -> torch.Tensor:
    """Keys and values expanded per head from one normed latent per token, plus one rotated key part that all heads
    share; a sink in the softmax; a gate per head."""
    t = h.shape[0]
    nh, d, r, dv, rank = int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"]), int(m["kv_rank"])
    pos = torch.arange(t, dtype=F)
    q = (h @ w[pre + ".q"].T).view(t, nh, d + r)
    dkv = h @ w[pre + ".dkv"].T
    c = plain_norm(dkv[:, :rank], w[pre + ".dkv.norm"], eps)
    k_rot = rotate_halves(dkv[:, rank:], pos, m["rot"])  # [T, r]
    q_rot = rotate_halves(q[..., d:], pos, m["rot"])  # [T, H, r]
    k_plain = (c @ w[pre + ".uk"].T).view(t, nh, d)
    v = (c @ w[pre + ".uv"].T).view(t, nh, dv)
    scores = (torch.einsum("ihd,jhd->hij", q[..., :d], k_plain) + torch.einsum("ihr,jr->hij", q_rot, k_rot)) * float(m["scale"])
    p = causal_softmax(scores, w[pre + ".sink"])
    o = torch.einsum("hij,jhd->ihd", p, v)
    gate = torch.sigmoid(h @ w[pre + ".g"].T)
    return (o * gate[:, :, None]).reshape(t, nh * dv) @ w[pre + ".o"].T


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def gated_ff(h: torch.Tensor, w: dict, pre: str) -> torch.Tensor:
    return (silu(h @ w[pre + ".gate"].T) * (h @ w[pre + ".up"].T)) @ w[pre + ".down"].T


def routed_ff(h: torch.Tensor, mlp: dict, w: dict, pre: str, gaps: list | None = None) -> torch.Tensor:
    """Every token: the ``top`` experts of the largest router logits, weighted by the softmax over those logits. ``gaps``
    collects, per token, how far the last picked logit lies above the first one left out, as a share of the largest."""
    top = int(mlp["router"]["top"])
    z = h @ w[pre + ".router"].T
    val, idx = torch.topk(z, top, dim=-1)
    if gaps is not None and top < z.shape[-1]:
        ranked = z.sort(dim=-1, descending=True).values
        gaps.append((ranked[:, top - 1] - ranked[:, top]) / z.abs().amax(dim=-1))
    wt = torch.softmax(val, dim=-1)
    out = torch.zeros(h.shape[0], w[pre + ".e0.down"].shape[0], dtype=F)
    for t in range(h.shape[0]):
        for j in range(top):
            out[t] += wt[t, j] * gated_ff(h[t:t + 1], w, f"{pre}.e{int(idx[t, j])}")[0]
    return out


MIXERS = {"attention": softmax_attention, "latent_attention": latent_attention}


def forward(cfg: dict, w: dict, tokens: list[int], layer_outputs: list | None = None, router_gaps: list | None = None,
            after_norm=None) -> torch.Tensor:
    """Logits [T, vocab] of a whole sequence; ``layer_outputs`` collects the sum of the streams behind every layer,
    ``router_gaps`` every routed layer's gaps (:func:`routed_ff`); ``after_norm`` (a function) is applied to every part's
    normed input (a rounding, to see how far a sequence's logits move under it)."""
    after_norm = after_norm or (lambda z: z)
    eps, s = float(cfg["norm"]["eps"]), int(cfg.get("streams", 1))
    x = w["embed"][torch.tensor(tokens, dtype=torch.long)]
    streams = x[None].repeat(s, 1, 1)
    for i, layer in enumerate(cfg["layers"]):
        pre = f"l{i}"
        u = streams_read(streams, w[pre + ".hc1.in"])
        y = MIXERS[layer["type"]](after_norm(offset_norm(u, w[pre + ".norm1"], eps)), layer["mixer"], w, pre + ".mix", eps)
        streams = streams_write(streams, y, w[pre + ".hc1.mix"], w[pre + ".hc1.out"])
        mlp = layer.get("mlp")
        if mlp is not None:
            u = streams_read(streams, w[pre + ".hc2.in"])
            hn = after_norm(offset_norm(u, w[pre + ".norm2"], eps))
            y = gated_ff(hn, w, pre + ".mlp") if mlp["kind"] == "dense" else routed_ff(hn, mlp, w, pre + ".mlp", router_gaps)
            streams = streams_write(streams, y, w[pre + ".hc2.mix"], w[pre + ".hc2.out"])
        if layer_outputs is not None:
            layer_outputs.append(streams.sum(dim=0))
    return offset_norm(streams.sum(dim=0), w["final.norm"], eps) @ w["head"].T
