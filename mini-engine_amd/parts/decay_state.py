"""Linear attention with a fixed decay per head and a matrix of state per request and head.

Per head, with q, k of ``key_dim`` and v of ``value_dim`` elements::

    S_t = decay_h * S_(t-1) + k_t v_t^T,     o_t = S_t^T q_t

There is no softmax and no denominator. ``S`` starts at zero, is float32, and lives in the request's state slot
between steps. One product gives q, k, v and the gate (the four weights are stacked at load time); the kernels of
``csrc/decay_state.hip`` then apply the spec's activation to q, k and v, rotate the first elements of q and k by the
position's angles (if the spec has a position encoding), scale k, walk the new tokens from the state, norm the
outputs (every head by its own root mean square, or all heads together with a weight), and multiply by the gate's
activation; the output projection follows. Sizes, decays, activations, scale, eps and the kind of the output norm all
come from the spec.
"""

from __future__ import annotations

import numpy as np
import torch

from ..ops import kernels as K
from ..weights.loader import TensorWant
from .base import MIXERS, POSITION_ENCODINGS, Mixer, StateBinding, StateNeed

INPUT_ACTIVATIONS = {"none": 0, "silu": 1}
GATE_ACTIVATIONS = {"silu": 1, "sigmoid": 2}
OUTPUT_NORMS = {"per_head": 0, "all_heads": 1}
MAX_KEY_DIM = 256


class DecayState(Mixer):
    graph_safe = True

    def __init__(self, spec, dtype, device):
        super().__init__(spec, dtype, device)
        s = spec
        for what, table, name in ((s.input_activation, INPUT_ACTIVATIONS, "input_activation"),
                                  (s.gate_activation, GATE_ACTIVATIONS, "gate_activation"),
                                  (s.output_norm, OUTPUT_NORMS, "output_norm")):
            if what not in table:
                raise ValueError(f"decay_state knows {name} in {sorted(table)}, got {what!r}")
        if len(s.decay) != s.num_heads:
            raise ValueError(f"{len(s.decay)} decays for {s.num_heads} heads")
        if not all(0.0 <= float(v) <= 1.0 for v in s.decay):
            raise ValueError("a decay lies in [0, 1]")
        if not (1 <= s.key_dim <= MAX_KEY_DIM and s.value_dim >= 1 and 1 <= s.num_heads <= 256):
            raise ValueError(f"decay_state takes up to 256 heads and keys of up to {MAX_KEY_DIM} elements, "
                             f"got {s.num_heads} heads of {s.key_dim} x {s.value_dim}")
        self.h, self.d, self.dv = int(s.num_heads), int(s.key_dim), int(s.value_dim)
        self.position = None if s.position is None else POSITION_ENCODINGS.build(s.position, dtype, device)
        if self.position is not None and self.position.rotary_dim > self.d:
            raise ValueError(f"{self.position.rotary_dim} rotated elements of a key of {self.d}")
        self.pairing = 0 if self.position is None else int(getattr(self.position, "pairing_code", 0))
        # the decay as two floats: the nearest float, and what that misses of the configured value
        hi = np.asarray(s.decay, dtype=np.float64).astype(np.float32)
        lo = (np.asarray(s.decay, dtype=np.float64) - hi.astype(np.float64)).astype(np.float32)
        self.decay = torch.from_numpy(np.stack((hi, lo))).to(device)
        names = dict(getattr(s, "names", ()) or ())
        self._n = {r: names.get(r, d) for r, d in (("q", "q_proj.weight"), ("k", "k_proj.weight"), ("v", "v_proj.weight"),
                                                    ("g", "g_proj.weight"), ("o", "o_proj.weight"), ("norm", "norm.weight"))}
        self.w_qkvg = self.w_o = self.norm_w = None

    # ---- weights
    def weight_wants(self, prefix: str) -> dict[str, TensorWant]:
        s, n = self.spec, self._n
        wants = {
            f"{prefix}.{n['q']}": TensorWant((self.h * self.d, s.hidden_size)),
            f"{prefix}.{n['k']}": TensorWant((self.h * self.d, s.hidden_size)),
            f"{prefix}.{n['v']}": TensorWant((self.h * self.dv, s.hidden_size)),
            f"{prefix}.{n['g']}": TensorWant((self.h * self.dv, s.hidden_size)),
            f"{prefix}.{n['o']}": TensorWant((s.hidden_size, self.h * self.dv)),
        }
        if s.output_norm == "all_heads":
            wants[f"{prefix}.{n['norm']}"] = TensorWant((self.h * self.dv,), "vector")
        return wants

    def load(self, tensors, prefix: str) -> None:
        n = self._n
        self.w_qkvg = torch.cat([tensors[f"{prefix}.{n[r]}"] for r in ("q", "k", "v", "g")], dim=0)
        self.w_o = tensors[f"{prefix}.{n['o']}"]
        if self.spec.output_norm == "all_heads":
            self.norm_w = tensors[f"{prefix}.{n['norm']}"]

    # ---- state
    def cache_need(self):
        return StateNeed((self.h, self.d, self.dv), torch.float32)

    # ---- step
    def _codes(self):
        s = self.spec
        return INPUT_ACTIVATIONS[s.input_activation], OUTPUT_NORMS[s.output_norm], GATE_ACTIVATIONS[s.gate_activation]

    def forward(self, h, batch, cache: StateBinding | None = None) -> torch.Tensor:
        if cache is None:
            raise RuntimeError("decay_state mixer was given no state")
        s = self.spec
        in_act, norm_kind, gate_act = self._codes()
        proj = K.linear(h, self.w_qkvg)
        rope = None if self.position is None else self.position.tables(batch.max_ctx)
        out = K.decay_state(proj, rope, self.pairing, batch.positions, self.decay, self.norm_w, cache.state, batch.item_start,
                            batch.state_slots, self.h, self.d, self.dv, in_act, float(s.key_scale), norm_kind, gate_act,
                            float(s.norm_eps), longest_item=0 if batch.decode_only else int(batch.max_qlen))
        return K.linear(out, self.w_o, as_delta=True)

    def emit(self, program, h, cache: StateBinding | None = None) -> None:
        if cache is None:
            raise RuntimeError("decay_state mixer was given no state")
        s = self.spec
        in_act, norm_kind, gate_act = self._codes()
        proj = program.linear(h, self.w_qkvg)
        out = program.decay_state(
            proj, decay=self.decay, rope=None if self.position is None else self.position.tables(program.max_positions),
            pairing=self.pairing, norm_weight=self.norm_w, state=cache.state, heads=self.h, key_dim=self.d, value_dim=self.dv,
            input_act=in_act, key_scale=float(s.key_scale), norm_kind=norm_kind, gate_act=gate_act, eps=float(s.norm_eps))
        program.linear_delta(out, self.w_o)


MIXERS.register("decay_state", DecayState)
