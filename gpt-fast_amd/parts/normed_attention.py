"""Causal attention over the paged cache with per-head normed queries and keys, a rotation of
part of each head, capped scores and a sliding window."""
import torch

from ..cache.store import KVNeed
from ..config.spec import NormedAttentionSpec
from ..ops import linear as L
from ..ops import scored_attention as SA
from .base import Param, Part, Runtime, add_late, check_bound, register_mixer
from .position import RotaryPosition, frequencies_and_trig_scale


class NormedAttention(Part):
    """q, k, v = split(wqkv x); every head of q and k is divided by its root mean square and
    multiplied by a weight that the heads share (``q_norm``, ``k_norm`` of ``head_dim``
    elements); the first ``rotary_dim`` elements of every head of q and k are rotated (pair
    layout, frequency ladder and the factor on cos and sin are the position spec's); for query
    i and key j with ``0 <= i - j < window``: ``s = (q . k) scale``, capped by ``softcap tanh(s /
    softcap)``; softmax over j; the values of kv head ``h // (H / G)``; then ``wo``.  The
    projection keeps its float32 sums until q and k are normed and rotated; scores, softmax and
    the weighted sums are float32.  The cache holds the normed, rotated keys; a windowed cache
    group gives pages back once every key in them is out of reach."""

    libraries = ("scored_attention",)
    replayable = True
    defers_sum = True              # ``residual`` may be a parts.base.ResidualStream

    def __init__(self, spec: NormedAttentionSpec, runtime: Runtime):
        if spec.n_heads % spec.n_kv_heads:
            raise ValueError(f"{spec.n_heads} heads do not divide into {spec.n_kv_heads} kv heads")
        if spec.window is not None and spec.window < 1:
            raise ValueError(f"a window of {spec.window} keys")
        self.spec = spec
        self.rt = runtime
        s = spec
        self.in_rows = (s.n_heads + s.n_kv_heads) * s.head_dim + s.n_kv_heads * s.value_dim
        self.rotary_dim, self.layout, self.freqs, self.trig = 0, 0, None, 1.0
        if s.position is not None and s.position.kind == "rope" and s.position.rotary_dim:
            if s.position.rotary_dim > s.head_dim:
                raise ValueError(f"{s.position.rotary_dim} rotated elements in heads of {s.head_dim}")
            freqs, self.trig = frequencies_and_trig_scale(s.position)
            self.freqs = freqs.to(runtime.device)
            self.rotary_dim = s.position.rotary_dim
            self.layout = RotaryPosition.LAYOUTS[s.position.layout]
        elif s.position is not None and s.position.kind not in ("rope", "none"):
            raise ValueError(f"normed attention takes rope or no position, not '{s.position.kind}'")
        self.wqkv = self.wo = self.q_norm = self.k_norm = None

    def parameters(self):
        s = self.spec
        p = {"wqkv": Param((self.in_rows, s.dim)), "wo": Param((s.dim, s.n_heads * s.value_dim))}
        if s.qk_norm_eps is not None:
            p["q_norm"] = Param((s.head_dim,), role="vector", init="norm")
            p["k_norm"] = Param((s.head_dim,), role="vector", init="norm")
        return p

    def bind(self, tensors):
        check_bound("NormedAttention", self.parameters(), tensors)
        # zero rows up to a multiple of eight: the products' kernels store whole groups
        self.wqkv, self.wo = L.pad_rows(tensors["wqkv"], 8), tensors["wo"]
        f32 = lambda name: tensors[name].to(torch.float32).contiguous() if name in tensors else None
        self.q_norm, self.k_norm = f32("q_norm"), f32("k_norm")

    def cache_need(self):
        s = self.spec
        return KVNeed(s.n_kv_heads, s.head_dim, s.window, s.value_dim)

    def step_flops(self, q_lens, starts) -> float:
        s = self.spec
        flops = 2.0 * sum(q_lens) * (self.in_rows + s.n_heads * s.value_dim) * s.dim
        for q, start in zip(q_lens, starts):
            keys = q * start + q * (q + 1) / 2.0
            if s.window is not None:
                keys = min(keys, q * s.window)
            flops += 2.0 * s.n_heads * (s.head_dim + s.value_dim) * keys
        return flops

    def _heads(self, x, batch, entry):
        s = self.spec
        proj = L.linear(x, self.wqkv, out_dtype=torch.float32)
        write = entry is not None and entry.writes
        table = batch.table(entry.group_id)
        q = SA.unit_heads_store(proj, None, batch.tok_seq, batch.tok_pos, table,
                                entry.k_pages if write else None, entry.v_pages if write else None,
                                s.n_heads, s.n_kv_heads, s.head_dim, s.value_dim, s.qk_norm_eps,
                                self.rt.dtype, q_weight=self.q_norm, k_weight=self.k_norm,
                                freqs=self.freqs, rotary_dim=self.rotary_dim, layout=self.layout,
                                trig_scale=self.trig)
        y = SA.attention(q, entry.k_pages, entry.v_pages, batch.tok_seq, batch.tok_pos, table,
                         s.scale, window=s.window or 0, softcap=s.softcap or 0.0,
                         step=(batch.q_start, batch.start_pos, batch.n_seqs, batch.max_q_len))
        return y.view(q.shape[0], s.n_heads * s.value_dim)

    def forward(self, x, batch, entry, residual):
        y = self._heads(x, batch, entry)
        add_late(residual, lambda rows, then_norm, takes_halves: L.linear_into(
            y, self.wo, rows, then_norm, takes_halves))

    def forward_rows(self, x, batch, entry):
        """The mixer's output alone: the output projection's float32 sums."""
        return L.linear(self._heads(x, batch, entry), self.wo, out_dtype=torch.float32)


register_mixer("normed_attention", NormedAttention)
