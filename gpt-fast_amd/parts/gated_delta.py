"""Recurrent mixer with the gated delta rule behind short causal convolutions."""
import dataclasses

import torch

from ..cache.store import StateNeed
from ..config.spec import GatedDeltaSpec
from ..ops import decayed_memory as DM
from ..ops import gated_delta as GD
from ..ops import linear as L
from .base import Param, Part, Runtime, add_late, check_bound, register_mixer


class GatedDelta(Part):
    """Per head a state ``S [dk, dv]``, float32, zero at a sequence's start, kept in the cache's
    state slot of the sequence together with the convolutions' last inputs:

        q, k, v = silu(conv(w x))                         (a causal convolution per channel)
        q = q / |q| * dk^-1/2     k = k / |k|             (per head; |.| with unit_eps inside)
        beta = sigmoid(w_b x)     g = exp(-exp(A_log) softplus(w_a x + dt_bias))
        S <- g S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q

    then each head's o over its root mean square, times ``norm`` (shared by the heads), times
    silu(w_g x), then ``wo``.  The input projections are one matrix ``w_in`` (rows of q, k, v,
    beta, the decay, the gate) whose product keeps its float32 sums: the convolutions, the
    gates, the state and everything up to the operand of ``wo`` are float32 whatever the
    engine's type."""

    replayable = True
    libraries = ("gated_delta", "decayed_memory")
    defers_sum = True              # ``residual`` may be a parts.base.ResidualStream

    def __init__(self, spec: GatedDeltaSpec, runtime: Runtime):
        s = spec
        if s.n_heads % s.n_kv_heads:
            raise ValueError(f"gated delta: {s.n_heads} heads do not divide into {s.n_kv_heads} key heads")
        if s.key_dim > GD.MAX_KEY_DIM or not 1 <= s.conv_taps <= GD.MAX_TAPS:
            raise ValueError(f"gated delta: key_dim {s.key_dim} (up to {GD.MAX_KEY_DIM}), "
                             f"{s.conv_taps} taps (1..{GD.MAX_TAPS})")
        self.spec = spec
        self.rt = runtime
        rows = GD.RowLayout.fused(s.n_heads, s.n_kv_heads, s.key_dim, s.value_dim)
        self.in_rows = rows.width                       # rows of w_in as it is stored
        self.rows = dataclasses.replace(rows, width=(rows.width + 7) // 8 * 8)
        self.tail_offset = s.n_heads * s.key_dim * s.value_dim
        self.w_in = self.wo = self.taps = self.norm = self.A_log = self.dt_bias = None

    def parameters(self):
        s = self.spec
        return {"w_in": Param((self.in_rows, s.dim)),
                "taps": Param((self.rows.conv, s.conv_taps), role="vector", init="unit"),
                "A_log": Param((s.n_heads,), role="vector", init="around_zero"),
                "dt_bias": Param((s.n_heads,), role="vector", init="around_zero"),
                "norm": Param((s.value_dim,), role="vector", init="norm"),
                "wo": Param((s.dim, s.n_heads * s.value_dim))}

    def bind(self, tensors):
        check_bound("GatedDelta", self.parameters(), tensors)
        # zero rows up to a multiple of eight: the products' kernels store whole groups
        self.w_in, self.wo = L.pad_rows(tensors["w_in"], 8), tensors["wo"]
        f32 = lambda name: tensors[name].to(torch.float32).contiguous()
        self.taps, self.norm, self.A_log, self.dt_bias = f32("taps"), f32("norm"), f32("A_log"), f32("dt_bias")

    def cache_need(self):
        s = self.spec
        return StateNeed((GD.state_size(s.n_heads, s.n_kv_heads, s.key_dim, s.value_dim, s.conv_taps),),
                         "float32")

    def step_flops(self, q_lens, starts) -> float:
        s = self.spec
        n = sum(q_lens)
        cell = 2.0 * 3.0 * s.n_heads * s.key_dim * s.value_dim          # two reads and the update of S
        return n * (2.0 * (self.in_rows + s.n_heads * s.value_dim) * s.dim + cell
                    + 2.0 * self.rows.conv * s.conv_taps)

    def _gated(self, x, batch, entry):
        s = self.spec
        proj = L.linear(x, self.w_in, out_dtype=torch.float32)
        conv = GD.short_conv(proj, self.rows, self.taps, entry.state, self.tail_offset, batch.tok_seq,
                             batch.q_start, batch.slots, batch.n_seqs)
        o = GD.cell(conv, proj, self.rows, self.A_log, self.dt_bias, entry.state, batch.q_start,
                    batch.slots, batch.n_seqs, batch.max_q_len, s.n_heads, s.n_kv_heads, s.key_dim,
                    s.value_dim, s.key_dim ** -0.5, s.unit_eps)
        return DM.row_norm_gate(o, self.norm, proj, self.rows, s.eps, self.rt.dtype,
                                groups=s.n_heads, gate="silu")

    def forward(self, x, batch, entry, residual):
        y = self._gated(x, batch, entry)
        add_late(residual, lambda rows, then_norm, takes_halves: L.linear_into(
            y, self.wo, rows, then_norm, takes_halves))

    def forward_rows(self, x, batch, entry):
        """The mixer's output alone: the output projection's float32 sums."""
        return L.linear(self._gated(x, batch, entry), self.wo, out_dtype=torch.float32)


register_mixer("gated_delta", GatedDelta)
