"""A plain, slow Gonurax in double precision on the CPU: one function per mechanism, token by token where the
mechanism is a recurrence, whole score matrices where it is attention. It shares no code with the package; the
tests hold the engine against it.

``cfg`` is the dictionary of a ``config.json``; ``w`` maps tensor names to tensors (any float dtype).

Notation: ``x`` the residual stream ``[T, width]``, ``h`` a layer's normed input, ``p`` absolute positions
``[T]``. Everything works on one sequence; a continuation takes the ``state`` (a dict per layer) that the call
before returned, so that prefill, decoding and any way of cutting can be compared.
"""

from __future__ import annotations

import math

import torch

F64 = torch.float64


def grouped_rms_norm(x: torch.Tensor, weight: torch.Tensor, groups: int, eps: float) -> torch.Tensor:
    """Each of ``groups`` equal consecutive parts of the last axis over its own sqrt(mean(part^2) + eps); the whole
    times ``weight``."""
    t, n = x.shape
    parts = x.reshape(t, groups, n // groups)
    parts = parts / torch.sqrt((parts * parts).mean(dim=-1, keepdim=True) + eps)
    return parts.reshape(t, n) * weight.to(F64)


def unit_rms(x: torch.Tensor, eps: float) -> torch.Tensor:
    return x / torch.sqrt((x * x).mean(dim=-1, keepdim=True) + eps)


def gelu_tanh(z: torch.Tensor) -> torch.Tensor:
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z**3)))


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def rotate_pairs(v: torch.Tensor, p: torch.Tensor, dims: int, base: float, layout: str, sign: float = 1.0) -> torch.Tensor:
    """``v`` ``[T, heads, n]``: its first ``dims`` elements turned by ``sign * p * base^(-2i/dims)``, pair ``i`` being
    ``(i, i + dims/2)`` ("halves") or ``(2i, 2i + 1)`` ("interleaved"); the rest unchanged."""
    half = dims // 2
    freq = torch.tensor([base ** (-2.0 * i / dims) for i in range(half)], dtype=F64)
    ang = sign * p.to(F64)[:, None] * freq[None, :]  # [T, half]
    cos, sin = torch.cos(ang)[:, None, :], torch.sin(ang)[:, None, :]
    out = v.clone()
    if layout == "halves":
        a, b = v[..., :half], v[..., half:dims]
        out[..., :half] = a * cos - b * sin
        out[..., half:dims] = b * cos + a * sin
    elif layout == "interleaved":
        a, b = v[..., 0:dims:2], v[..., 1:dims:2]
        out[..., 0:dims:2] = a * cos - b * sin
        out[..., 1:dims:2] = b * cos + a * sin
    else:
        raise ValueError(layout)
    return out


def visible(i: int, j: int, size: int, keep_first: int) -> bool:
    return j <= i and (i - j < size or j < keep_first)


def window_attention(h, p, w, prefix, m, eps, state):
    """Softmax attention with grouped key/value heads, per-head q/k norm, interleaved rotation of q and k, values
    rotated by their own position and the output turned back by the query's, a sliding window that keeps the first
    tokens. ``state``: all keys, rotated values and positions so far."""
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    t = h.shape[0]
    q = (h @ w[f"{prefix}.q"].to(F64).T).reshape(t, H, d)
    k = (h @ w[f"{prefix}.k"].to(F64).T).reshape(t, G, d)
    v = (h @ w[f"{prefix}.v"].to(F64).T).reshape(t, G, dv)
    q = unit_rms(q, eps) * w[f"{prefix}.q.norm"].to(F64)
    k = unit_rms(k, eps) * w[f"{prefix}.k.norm"].to(F64)
    rot = m["rot"]
    q = rotate_pairs(q, p, rot["dims"], rot["base"], "interleaved")
    k = rotate_pairs(k, p, rot["dims"], rot["base"], "interleaved")
    v = rotate_pairs(v, p, dv, rot["base"], "interleaved")
    if state is not None:
        k = torch.cat((state["k"], k))
        v = torch.cat((state["v"], v))
        pk = torch.cat((state["p"], p))
    else:
        pk = p
    size, keep = m["mask"]["size"], m["mask"]["keep_first"]
    out = torch.zeros(t, H, dv, dtype=F64)
    for a in range(t):
        i = int(p[a])
        js = [b for b in range(pk.shape[0]) if visible(i, int(pk[b]), size, keep)]
        for head in range(H):
            g = head // (H // G)
            s = (k[js, g] @ q[a, head]) * m["scale"]
            pr = torch.softmax(s, dim=0)
            out[a, head] = pr @ v[js, g]
    out = rotate_pairs(out, p, dv, rot["base"], "interleaved", sign=-1.0)
    y = out.reshape(t, H * dv) @ w[f"{prefix}.o"].to(F64).T
    return y, {"k": k, "v": v, "p": pk}


def decayed_state_scan(q, k, v, decay, s0):
    """Per head ``S_t = decay_h S_(t-1) + k_t v_t^T`` and ``o_t = S_t^T q_t``, token by token. q, k ``[T, H, d]``,
    v ``[T, H, dv]``, s0 ``[H, d, dv]`` or None."""
    t, H, d = q.shape
    dv = v.shape[-1]
    S = torch.zeros(H, d, dv, dtype=F64) if s0 is None else s0.clone()
    lam = torch.tensor(decay, dtype=F64)[:, None, None]
    out = torch.zeros(t, H, dv, dtype=F64)
    for a in range(t):
        S = lam * S + k[a][:, :, None] * v[a][:, None, :]
        out[a] = torch.einsum("hij,hi->hj", S, q[a])
    return out, S


def retention(h, p, w, prefix, m, eps, state):
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    t = h.shape[0]
    q = (h @ w[f"{prefix}.q"].to(F64).T).reshape(t, H, d)
    k = (h @ w[f"{prefix}.k"].to(F64).T).reshape(t, H, d)
    v = (h @ w[f"{prefix}.v"].to(F64).T).reshape(t, H, dv)
    rot = m["rot"]
    q = rotate_pairs(q, p, rot["dims"], rot["base"], "halves")
    k = rotate_pairs(k, p, rot["dims"], rot["base"], "halves") * d**-0.5
    o, S = decayed_state_scan(q, k, v, m["decay"], None if state is None else state["S"])
    o = unit_rms(o, eps).reshape(t, H * dv)
    o = o * silu(h @ w[f"{prefix}.g"].to(F64).T)
    return o @ w[f"{prefix}.o"].to(F64).T, {"S": S}


def lightning(h, p, w, prefix, m, eps, state):
    H, d, dv = m["heads"], m["dim"], m["vdim"]
    t = h.shape[0]
    q = silu(h @ w[f"{prefix}.q"].to(F64).T).reshape(t, H, d)
    k = silu(h @ w[f"{prefix}.k"].to(F64).T).reshape(t, H, d)
    v = silu(h @ w[f"{prefix}.v"].to(F64).T).reshape(t, H, dv)
    o, S = decayed_state_scan(q, k, v, m["decay"], None if state is None else state["S"])
    o = unit_rms(o.reshape(t, H * dv), eps) * w[f"{prefix}.norm"].to(F64)
    o = o * torch.sigmoid(h @ w[f"{prefix}.g"].to(F64).T)
    return o @ w[f"{prefix}.o"].to(F64).T, {"S": S}


MIXERS = {"attention": window_attention, "retention": retention, "lightning": lightning}


def dense_ff(h, w, prefix):
    return (gelu_tanh(h @ w[f"{prefix}.gate"].to(F64).T) * (h @ w[f"{prefix}.up"].to(F64).T)) @ w[f"{prefix}.down"].to(F64).T


def forward(cfg: dict, w: dict, tokens, start: int = 0, states=None, layers_out: list | None = None):
    """Logits ``[T, vocab]`` (double) of ``tokens`` at positions ``start ..`` and the states to continue from."""
    eps, groups, mult = cfg["norm"]["eps"], cfg["norm"]["groups"], cfg["residual_mult"]
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    p = torch.arange(start, start + tokens.shape[0])
    x = w["embed"].to(F64)[tokens]
    new_states = []
    for i, layer in enumerate(cfg["layers"]):
        h = grouped_rms_norm(x, w[f"l{i}.norm1"], groups, eps)
        y, st = MIXERS[layer["type"]](h, p, w, f"l{i}.mix", layer["mixer"], eps, None if states is None else states[i])
        if layer.get("mlp") is not None:
            y = y + dense_ff(h, w, f"l{i}.mlp")
        x = x + mult * y
        new_states.append(st)
        if layers_out is not None:
            layers_out.append(x.clone())
    x = grouped_rms_norm(x, w["final.norm"], groups, eps)
    return x @ w["embed"].to(F64).T, new_states


def forward_in_portions(cfg, w, tokens, cuts):
    """The same logits, the sequence fed in portions that end at ``cuts`` (and at its end)."""
    outs, states, at = [], None, 0
    for end in list(cuts) + [len(tokens)]:
        if end <= at:
            continue
        lg, states = forward(cfg, w, tokens[at:end], at, states)
        outs.append(lg)
        at = end
    return torch.cat(outs)
