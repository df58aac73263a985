"""The gated delta rule: a recurrent mixer with a matrix state per head."""
from __future__ import annotations

from typing import Dict, Optional

import torch

from .. import ops
from ..config.forward_config import PartSpec
from ..weights.loader import WeightSpec
from .base import LayerMemory, Mixer, Runtime, StateRequest, register_mixer
from .rows import ProductRows


@register_mixer("gated_delta_rule")
class GatedDeltaRule(Mixer):
    """Per head a state S [dim, vdim] (float32, zero at a sequence's start), updated token by token:

        S <- g S;   u = beta (v - S^T k);   S <- S + k u^T;   o = S^T q      (the read-out sees the token's write)

    q and k [kv_heads, dim] and v [heads, vdim] are projections of x that pass a short causal convolution over
    time (per channel, ``conv`` taps, no bias, zeros before the start) and SiLU; q and k are then made unit vectors
    per head (x / sqrt(sum x^2 + 1e-6)), q also times dim^-1/2; head h reads q/k head h // (heads / kv_heads).
    beta = sigmoid(W_b x) and the decay g = exp(-exp(A_log) softplus(W_a x + dt_bias)), one of each per head.
    The output per head is o / rms(o) * w [vdim] * silu(W_g x), then W_o.

    A request's state is S and the last conv - 1 rows that entered the convolution, in one float32 row of the
    state slot.  The six projections are one stacked product with float32 results; everything after it up to the
    output projection is float32 arithmetic (``csrc/delta.hip``).  Steps of such a model are never padded.

    params: hidden_size, heads, kv_heads, dim, vdim, conv, eps."""

    graph_safe = True
    tape_safe = True
    padding_safe = False      # a padding token would move the state
    writes_into = True

    @staticmethod
    def weight_specs(spec: PartSpec) -> Dict[str, WeightSpec]:
        p = spec.params
        H, nh, kvh, dim, vdim, taps = (int(p[k]) for k in ("hidden_size", "heads", "kv_heads", "dim", "vdim", "conv"))
        return {"q": WeightSpec((kvh * dim, H)), "q_conv": WeightSpec((kvh * dim, taps)),
                "k": WeightSpec((kvh * dim, H)), "k_conv": WeightSpec((kvh * dim, taps)),
                "v": WeightSpec((nh * vdim, H)), "v_conv": WeightSpec((nh * vdim, taps)),
                "b": WeightSpec((nh, H)), "a": WeightSpec((nh, H)), "A_log": WeightSpec((nh,), init="zeros"),
                "dt_bias": WeightSpec((nh,), init="zeros"), "norm": WeightSpec((vdim,), init="ones"),
                "g": WeightSpec((nh * vdim, H)), "o": WeightSpec((H, nh * vdim))}

    def __init__(self, spec: PartSpec, weights: Dict[str, torch.Tensor], rt: Runtime):
        super().__init__(spec, weights, rt)
        p = spec.params
        self.hidden, self.nh, self.kvh, self.dim, self.vdim, self.taps = (
            int(p[k]) for k in ("hidden_size", "heads", "kv_heads", "dim", "vdim", "conv"))
        self.eps = float(p.get("eps", 1e-6))
        if self.nh % self.kvh:
            raise ValueError(f"gated_delta_rule: {self.nh} heads are not a multiple of {self.kvh} q/k heads")
        if not (1 <= self.taps <= ops.mixing.DELTA_MAX_TAPS) or self.dim > 256:
            raise ValueError("gated_delta_rule: conv must lie in 1..17 and dim be at most 256")
        self.channels = 2 * self.kvh * self.dim + self.nh * self.vdim
        self.gate_at = self.channels
        width = self.channels + self.nh * self.vdim + 2 * self.nh
        mats = [weights[k] for k in ("q", "k", "v", "g", "b", "a")]
        dt = mats[0].dtype
        stacked = torch.zeros((-(-width // 8) * 8, self.hidden), dtype=dt, device=mats[0].device)   # rows to a multiple of 8
        at = 0
        for m in mats:
            stacked[at:at + m.shape[0]] = m.to(dt)
            at += m.shape[0]
        self.w_in = stacked
        self.width = width
        self.conv_w = torch.cat([weights[k].float() for k in ("q_conv", "k_conv", "v_conv")]).contiguous()
        self.a_log, self.dt_bias = weights["A_log"].float().contiguous(), weights["dt_bias"].float().contiguous()
        self.norm = weights["norm"].float().contiguous()
        self.o = weights["o"]

    def state_request(self) -> Optional[StateRequest]:
        return StateRequest((ops.delta_state_floats(self.nh, self.dim, self.vdim, self.kvh, self.taps),), torch.float32)

    def step_rows(self, rows: int, kind: str) -> int:
        return ProductRows.step_rows(rows, kind)

    def forward(self, x: torch.Tensor, batch, memory: LayerMemory, out=None) -> torch.Tensor:
        n, rt, nh, kvh, dim, vdim = x.shape[0], self.rt, self.nh, self.kvh, self.dim, self.vdim
        state = memory.state
        full = ops.linear(x, self.w_in, out=rt.buffer("delta_proj", (n, self.w_in.shape[0]), torch.float32))
        proj = full[:, :self.width]
        qk = rt.buffer("delta_qk", (n, 2 * kvh * dim), torch.float32)
        v = rt.buffer("delta_v", (n, nh * vdim), torch.float32)
        beta_g = rt.buffer("delta_beta_g", (n, 2, nh), torch.float32)
        ops.delta_prepare(proj, self.conv_w, self.a_log, self.dt_bias, state, batch.tok_seq, batch.entry_start,
                          batch.entry_slot, nh, kvh, dim, vdim, self.taps, qk, v, beta_g)
        ops.delta_conv_state(state, proj, batch.entry_start, batch.entry_len, batch.entry_slot, nh, kvh, dim, vdim,
                             self.taps)
        o = rt.buffer("delta_read", (n, nh * vdim), torch.float32)
        ops.delta_rule(qk, v, beta_g, state, batch.entry_start, batch.entry_len, batch.entry_slot, nh, kvh, dim, vdim, out=o)
        y = rt.buffer("delta_heads", (n, nh * vdim))
        ops.gated_rms_norm(o, self.norm, proj[:, self.gate_at:self.gate_at + nh * vdim], nh, vdim, self.eps, out=y)
        if out is None:
            out = rt.buffer("delta_out", (n, self.hidden))
        return ops.linear(y, self.o, out=out)
