"""Causal attention whose values are its keys, with a bias by the logarithm of the distance
and a sink in the softmax, over the paged cache."""
import torch

from ..cache.store import KVNeed
from ..config.spec import SinkAttentionSpec
from ..ops import linear as L
from ..ops import scored_attention as SA
from .base import Param, Part, Runtime, add_late, check_bound, register_mixer


class SinkAttention(Part):
    """``q, k = split(wqk x + bqk)``; a kv head's value is its key as projected (or, without
    ``values_are_keys``, a third part of the projection); all of q, and all of k, divided by
    the root mean square of the whole projection and multiplied by a weight per element; q at
    position p times ``1 + coef ln(floor((p + 1) / every) + 1)``; for query i, key j <= i and
    head h: ``s = (q_h . k_j) scale - r1[h] ln(1 + r2[h] (i - j))``; the softmax over j has one
    more term exp(0) in its denominator (a key of score zero without a value); the weights
    take the values of kv head ``h // (H / G)``; then ``wo``.  Each of these steps is a field
    of the spec.  The projection keeps its float32 sums until q and k are normed; positions,
    the temperature, scores, the bias, the softmax and the weighted sums are float32.  The
    cache holds the normed keys, and the values apart."""

    libraries = ("scored_attention",)
    replayable = True
    defers_sum = True              # ``residual`` may be a parts.base.ResidualStream

    def __init__(self, spec: SinkAttentionSpec, runtime: Runtime):
        if spec.n_heads % spec.n_kv_heads:
            raise ValueError(f"{spec.n_heads} heads do not divide into {spec.n_kv_heads} kv heads")
        if spec.values_are_keys and spec.value_dim != spec.head_dim:
            raise ValueError("values that are the keys have the keys' size")
        self.spec = spec
        self.rt = runtime
        s = spec
        self.nq, self.nk = s.n_heads * s.head_dim, s.n_kv_heads * s.head_dim
        self.in_rows = self.nq + self.nk + (0 if s.values_are_keys else s.n_kv_heads * s.value_dim)
        self.w_in = self.wo = self.b_in = None
        self.q_norm = self.k_norm = self.r1 = self.r2 = None

    def parameters(self):
        s = self.spec
        p = {"w_in": Param((self.in_rows, s.dim)), "wo": Param((s.dim, s.n_heads * s.value_dim))}
        if s.biases:
            p["b_in"] = Param((self.in_rows,), role="vector", init="around_zero")
        if s.whole_norm_eps is not None:
            p["q_norm"] = Param((self.nq,), role="vector", init="norm")
            p["k_norm"] = Param((self.nk,), role="vector", init="norm")
        if s.log_distance_bias:
            p["r1"] = Param((s.n_heads,), role="vector", init="norm")
            p["r2"] = Param((s.n_heads,), role="vector", init="norm")
        return p

    def bind(self, tensors):
        check_bound("SinkAttention", self.parameters(), tensors)
        # zero rows up to a multiple of eight: the products' kernels store whole groups
        self.w_in, self.wo = L.pad_rows(tensors["w_in"], 8), tensors["wo"]
        f32 = lambda name: tensors[name].to(torch.float32).contiguous() if name in tensors else None
        self.b_in, self.q_norm, self.k_norm = f32("b_in"), f32("q_norm"), f32("k_norm")
        self.r1, self.r2 = f32("r1"), f32("r2")

    def cache_need(self):
        s = self.spec
        return KVNeed(s.n_kv_heads, s.head_dim, None, s.value_dim)

    def step_flops(self, q_lens, starts) -> float:
        s = self.spec
        flops = 2.0 * sum(q_lens) * (self.in_rows + s.n_heads * s.value_dim) * s.dim
        for q, start in zip(q_lens, starts):
            keys = q * start + q * (q + 1) / 2.0
            flops += 2.0 * s.n_heads * (s.head_dim + s.value_dim) * keys
        return flops

    def _heads(self, x, batch, entry):
        s = self.spec
        proj = L.linear(x, self.w_in, out_dtype=torch.float32)
        write = entry is not None and entry.writes
        table = batch.table(entry.group_id)
        q = SA.whole_norm_store(proj, self.b_in, self.q_norm, self.k_norm, batch.tok_seq,
                                batch.tok_pos, table, entry.k_pages if write else None,
                                entry.v_pages if write else None, s.n_heads, s.n_kv_heads,
                                s.head_dim, s.value_dim, s.whole_norm_eps, s.q_temp_coef,
                                s.q_temp_every, s.values_are_keys, self.rt.dtype)
        y = SA.attention(q, entry.k_pages, entry.v_pages, batch.tok_seq, batch.tok_pos, table,
                         s.scale, log_bias=(self.r1, self.r2) if s.log_distance_bias else None,
                         sink=s.sink,
                         step=(batch.q_start, batch.start_pos, batch.n_seqs, batch.max_q_len))
        return y.view(q.shape[0], s.n_heads * s.value_dim)

    def forward(self, x, batch, entry, residual):
        y = self._heads(x, batch, entry)
        add_late(residual, lambda rows, then_norm, takes_halves: L.linear_into(
            y, self.wo, rows, then_norm, takes_halves))

    def forward_rows(self, x, batch, entry):
        """The mixer's output alone: the output projection's float32 sums."""
        return L.linear(self._heads(x, batch, entry), self.wo, out_dtype=torch.float32)


register_mixer("sink_attention", SinkAttention)
