"""Attention whose keys and values are expanded from one cached latent per token."""
import torch

from ..cache.store import KVNeed
from ..config.spec import LatentAttentionSpec
from ..ops import kernels as K
from ..ops import linear as L
from ..ops import scored_attention as SA
from .base import POSITIONS, Param, Part, Runtime, add_late, check_bound, register_mixer


class LatentAttention(Part):
    """``cq = norm(w_dq x)``, ``q = w_uq cq`` (per head ``d`` plain and ``dr`` rotated
    elements); ``[c', kr'] = w_dkv x``, ``c = norm(c')`` the token's latent, ``kr`` = kr'
    rotated by position, one key part for all heads.  A head's plain key is ``w_uk[h] c`` and
    its value ``w_uv[h] c``, so

        score_h(i, j) = (q_plain_h(i) . w_uk[h] c_j + q_rot_h(i) . kr_j) * scale
                      = ([w_uk[h]^T q_plain_h(i), q_rot_h(i)] . [c_j, kr_j]) * scale
        out_h(i) = w_uv[h] sum_j softmax_j(score_h)(i, j) c_j

    that is attention with one kv head whose key is ``[c, kr]`` and whose value is ``c``: the
    query is carried into the latent's space by ``w_uk`` before and the result out of it by
    ``w_uv`` after, one small product per head each.  The cache holds the latent (once in the
    order the kernels read keys in, once in the order they read values in) and the rotated
    part.  Keys at distance < ``window`` are seen.  The down projections keep their float32
    sums until the norms; the query's up projection keeps them until the rotation.

    Without a query latent (``q_rank`` None) ``q = w_q x``: the kv down projection and ``w_q``
    are then one matrix over x, whose float32 sums serve both."""

    libraries = ("scored_attention",)
    replayable = True
    defers_sum = True              # ``residual`` may be a parts.base.ResidualStream

    def __init__(self, spec: LatentAttentionSpec, runtime: Runtime):
        self.spec = spec
        self.rt = runtime
        self.position = POSITIONS.build(spec.position, runtime)
        if spec.position.kind == "rope":
            if spec.position.layout != "interleaved" or not hasattr(self.position, "freqs"):
                raise ValueError("latent attention rotates interleaved pairs by a frequency "
                                 "vector (position kind 'rope', layout 'interleaved')")
            self.rotary_dim, self.freqs = spec.position.rotary_dim, self.position.freqs
        elif spec.position.kind == "none":
            self.rotary_dim, self.freqs = 0, None
        else:
            raise ValueError(f"latent attention: position kind '{spec.position.kind}'")
        if self.rotary_dim > spec.rot_dim:
            raise ValueError(f"latent attention: {self.rotary_dim} rotated elements of {spec.rot_dim}")
        self.window = 0 if spec.window is None else int(spec.window)
        self.q_rank = int(spec.q_rank or 0)
        self.q_rows = spec.n_heads * (spec.head_dim + spec.rot_dim)
        # no query latent: [kv latent | rotated key part | q] over x
        self.down_rows = self.q_rank + spec.kv_rank + spec.rot_dim + (0 if self.q_rank else self.q_rows)
        self.w_down = self.w_uq = self.w_uk = self.w_uv = self.wo = None
        self.q_norm = self.kv_norm = None

    def parameters(self):
        s = self.spec
        p = {"w_down": Param((self.down_rows, s.dim)),
             "kv_norm": Param((s.kv_rank,), role="vector", init="norm"),
             "w_uk": Param((s.n_heads * s.head_dim, s.kv_rank)),
             "w_uv": Param((s.n_heads * s.value_dim, s.kv_rank)),
             "wo": Param((s.dim, s.n_heads * s.value_dim))}
        if self.q_rank:
            p["q_norm"] = Param((s.q_rank,), role="vector", init="norm")
            p["w_uq"] = Param((self.q_rows, s.q_rank))
        return p

    def bind(self, tensors):
        check_bound("LatentAttention", self.parameters(), tensors)
        s = self.spec
        # zero rows up to a multiple of eight: the products' kernels store whole groups
        self.w_down = L.pad_rows(tensors["w_down"], 8)
        self.w_uq = L.pad_rows(tensors["w_uq"], 8) if self.q_rank else None
        self.wo = tensors["wo"]
        # per head: [d, R] carries a plain query into the latent's space, [dv, R] a result out
        self.w_uk = tensors["w_uk"].view(s.n_heads, s.head_dim, s.kv_rank)
        self.w_uv = tensors["w_uv"].view(s.n_heads, s.value_dim, s.kv_rank)
        self.q_norm = tensors["q_norm"].to(torch.float32).contiguous() if self.q_rank else None
        self.kv_norm = tensors["kv_norm"].to(torch.float32).contiguous()

    def cache_need(self):
        s = self.spec
        return KVNeed(1, s.kv_rank + s.rot_dim, s.window, s.kv_rank)

    def step_flops(self, q_lens, starts) -> float:
        s = self.spec
        n = sum(q_lens)
        per_token = (self.down_rows * s.dim + self.q_rows * self.q_rank
                     + s.n_heads * (s.head_dim + s.value_dim) * s.kv_rank
                     + s.n_heads * s.value_dim * s.dim)
        flops = 2.0 * n * per_token
        for q, start in zip(q_lens, starts):
            keys = q * start + q * (q + 1) / 2.0
            if s.window is not None:
                keys = min(keys, q * float(s.window))
            flops += 2.0 * s.n_heads * (2 * s.kv_rank + s.rot_dim) * keys
        return flops

    def _per_head(self, a, w, out):
        """out[h] = a[h] w[h]^T for every head: a [H, N, K], w [H, M, K], out [H, N, M] (a view)."""
        if a.dtype == torch.float32:
            return K.gemm_f32_batched(a, w, out)
        return torch.bmm(a, w.transpose(1, 2), out=out)        # the vendor library, as for prompts

    def _heads(self, x, batch, entry):
        s = self.spec
        n = x.shape[0]
        R = s.kv_rank
        down = L.linear(x, self.w_down, out_dtype=torch.float32)
        write = entry is not None and entry.writes
        table = batch.table(entry.group_id)
        cq = SA.latent_store(down, self.q_rank, R, s.rot_dim, self.q_norm, self.kv_norm, s.eps,
                             self.freqs, self.rotary_dim, batch.tok_seq, batch.tok_pos, table,
                             entry.k_pages if write else None, entry.v_pages if write else None,
                             self.rt.dtype)
        if self.q_rank:
            q = L.linear(cq, self.w_uq, out_dtype=torch.float32)[:, :self.q_rows]
        else:
            q = down[:, R + s.rot_dim:R + s.rot_dim + self.q_rows]       # a view of the wider rows
        plain, full = SA.latent_query(q, self.freqs, self.rotary_dim, batch.tok_pos, s.n_heads,
                                      s.head_dim, s.rot_dim, R, self.rt.dtype)
        # w_uk[h] is [d, R]: as the second operand it is taken transposed, [R, d]
        self._per_head(plain, self.w_uk.transpose(1, 2), full[:, :, :R])
        latent = SA.attention(full, entry.k_pages, entry.v_pages, batch.tok_seq, batch.tok_pos,
                              table, s.scale, window=self.window, head_major=True,
                              step=(batch.q_start, batch.start_pos, batch.n_seqs, batch.max_q_len))
        y = torch.empty((n, s.n_heads, s.value_dim), dtype=self.rt.dtype, device=x.device)
        self._per_head(latent, self.w_uv, y.permute(1, 0, 2))
        return y.view(n, s.n_heads * s.value_dim)

    def forward(self, x, batch, entry, residual):
        y = self._heads(x, batch, entry)
        add_late(residual, lambda rows, then_norm, takes_halves: L.linear_into(
            y, self.wo, rows, then_norm, takes_halves))

    def forward_rows(self, x, batch, entry):
        """The mixer's output alone: the output projection's float32 sums."""
        return L.linear(self._heads(x, batch, entry), self.wo, out_dtype=torch.float32)


register_mixer("latent_attention", LatentAttention)
