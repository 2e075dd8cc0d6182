"""Linear attention with a fixed decay per head (lightning attention)."""
import dataclasses

import torch

from ..cache.store import StateNeed
from ..config.spec import DecayedMemorySpec
from ..ops import decayed_memory as M
from ..ops import kernels as K
from ..ops import linear as L
from .base import Param, Part, Runtime, add_late, check_bound, register_mixer
from .position import RotaryPosition, frequencies_and_trig_scale


class DecayedMemory(Part):
    """Per head a state ``S [dk, dv]``, float32, zero at a sequence's start, kept in the
    cache's state slot of the sequence and carried from step to step:

        q = act(w_q x)   k = act(w_k x)   v = act(w_v x)          (silu, or nothing)
        q, k rotated by their position; k times key_scale        (if the spec has a position)
        S' = decay_h S + k v^T          o = S'^T q

    then the heads' results over their root mean square (all heads side by side as one row,
    or every head by itself), times ``norm`` (if the spec has a weight), times sigmoid or silu
    of w_g x, then ``wo``.  The four input projections are one matrix ``w_in`` (rows of q, k,
    v, g) whose product keeps its float32 sums: the activations, the rotation, the state and
    everything up to the operand of ``wo`` are float32 whatever the engine's type."""

    replayable = True
    libraries = ("decayed_memory",)
    defers_sum = True              # ``residual`` may be a parts.base.ResidualStream

    def __init__(self, spec: DecayedMemorySpec, runtime: Runtime):
        if spec.key_dim > M.MAX_KEY_DIM:
            raise ValueError(f"decayed memory: key_dim {spec.key_dim} > {M.MAX_KEY_DIM}")
        if len(spec.decay) != spec.n_heads:
            raise ValueError(f"decayed memory: {len(spec.decay)} decays for {spec.n_heads} heads")
        if spec.activation not in ("silu", None) or spec.norm not in ("row", "head") \
                or spec.gate not in ("sigmoid", "silu"):
            raise ValueError(f"decayed memory: activation '{spec.activation}' (silu or None), norm "
                             f"'{spec.norm}' (row or head), gate '{spec.gate}' (sigmoid or silu)")
        self.rotary_dim, self.layout, self.freqs, self.trig = 0, 0, None, 1.0
        position = spec.position
        if position is not None and position.kind == "rope" and position.rotary_dim:
            if position.rotary_dim > spec.key_dim:
                raise ValueError(f"{position.rotary_dim} rotated elements in heads of {spec.key_dim}")
            freqs, self.trig = frequencies_and_trig_scale(position)
            self.freqs = freqs.to(runtime.device)
            self.rotary_dim = position.rotary_dim
            self.layout = RotaryPosition.LAYOUTS[position.layout]
        elif position is not None and position.kind not in ("rope", "none"):
            raise ValueError(f"decayed memory takes rope or no position, not '{position.kind}'")
        if (self.rotary_dim or spec.key_scale != 1.0) and spec.activation is not None:
            # the cell's kernels apply the activation themselves, after what is done to the rows
            raise ValueError("decayed memory: a rotation or key scale follows the projection "
                             "directly (activation None)")
        self.spec = spec
        self.rt = runtime
        rows = M.RowLayout.fused(spec.n_heads, spec.key_dim, spec.value_dim)
        self.in_rows = rows.width                       # rows of w_in as it is stored
        self.rows = dataclasses.replace(rows, width=(rows.width + 7) // 8 * 8)
        self.decay = torch.tensor(spec.decay, dtype=torch.float64).to(torch.float32).to(runtime.device)
        self.w_in = self.wo = self.norm = None

    def parameters(self):
        s = self.spec
        p = {"w_in": Param((self.in_rows, s.dim)), "wo": Param((s.dim, s.n_heads * s.value_dim))}
        if s.norm_weight:
            p["norm"] = Param((s.n_heads * s.value_dim,), role="vector", init="norm")
        return p

    def bind(self, tensors):
        check_bound("DecayedMemory", self.parameters(), tensors)
        # zero rows up to a multiple of eight: the products' kernels store whole groups
        self.w_in, self.wo = L.pad_rows(tensors["w_in"], 8), tensors["wo"]
        self.norm = tensors["norm"].to(torch.float32).contiguous() if "norm" in tensors else None

    def cache_need(self):
        s = self.spec
        return StateNeed((M.state_size(s.n_heads, s.key_dim, s.value_dim),), "float32")

    def step_flops(self, q_lens, starts) -> float:
        s = self.spec
        n = sum(q_lens)
        cell = 2.0 * 2.0 * s.n_heads * s.key_dim * s.value_dim          # update and read of S
        return n * (2.0 * (self.in_rows + s.n_heads * s.value_dim) * s.dim + cell)

    def _gated(self, x, batch, entry):
        s = self.spec
        proj = L.linear(x, self.w_in, out_dtype=torch.float32)
        if self.rotary_dim or s.key_scale != 1.0:
            # in place on the projection's float32 sums: the heads of q and, right behind them,
            # those of k with their factor
            assert self.rows.k == self.rows.q + s.n_heads * s.key_dim
            K.rotate_rows(proj, self.rows.q, 2 * s.n_heads, s.key_dim, self.rotary_dim, self.layout,
                          self.freqs, batch.tok_pos, self.trig, 1.0, late_from=s.n_heads,
                          late_factor=s.key_scale)
        o = M.cell(proj, self.rows, self.decay, entry.state, batch.q_start, batch.slots,
                   batch.n_seqs, batch.max_q_len, s.n_heads, s.key_dim, s.value_dim,
                   activation=s.activation is not None)
        return M.row_norm_gate(o, self.norm, proj, self.rows, s.eps, self.rt.dtype,
                               groups=s.n_heads if s.norm == "head" else 1, gate=s.gate)

    def forward(self, x, batch, entry, residual):
        y = self._gated(x, batch, entry)
        add_late(residual, lambda rows, then_norm, takes_halves: L.linear_into(
            y, self.wo, rows, then_norm, takes_halves))

    def forward_rows(self, x, batch, entry):
        """The mixer's output alone: the output projection's float32 sums."""
        return L.linear(self._gated(x, batch, entry), self.wo, out_dtype=torch.float32)


register_mixer("decayed_memory", DecayedMemory)
