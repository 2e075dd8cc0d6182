"""A mixture-of-experts feed-forward: a router chooses a few small feed-forwards per token."""
import torch

from ..config.spec import RoutedExpertsSpec
from ..ops import kernels as K
from ..ops import linear as L
from ..ops import routed_experts as RE
from .base import Param, Part, Runtime, check_bound, register_feed_forward

# steps of more rows than this put the (token, expert) pairs in the order of their experts and
# run one product per expert; single-token steps of any size and steps of fewer rows take the
# kernels that work pair by pair
PAIRWISE_MAX_ROWS = 16
# from this many rows on, bfloat16 steps of few rows put the pairs in the order of their experts
# on the device and read each expert's matrices once for all of its rows
GROUPED_MIN_ROWS = 1
# prompts: the experts' shares of the pairs are padded to the largest share (rounded up to this
# many rows) and all experts are one batched product, unless the padded rows are more than this
# many times the pairs (a router that sends most tokens to few experts): then one product per
# expert over its own rows
PAD_ROWS_TO = 32
PADDED_MAX_WASTE = 1.5


class RoutedExperts(Part):
    """``y = sum_k weight_k expert_{e_k}(x) + shared(x)`` with ``expert(x) = w_down act(w_up x)``
    or, for gated experts, ``w_down (act(w_gate x) * (w_up x))``.
    The router's logits are float32 sums of ``w_router x``; scores (softmax or sigmoid), the
    correction that only the choice sees, the groups' choice, the top experts and their
    weights are worked out in float32 by one kernel per step.  The experts' matrices are
    stacked, ``w_up [E, F, D]`` (gated: ``[E, 2 F, D]``, an expert's gate rows and then its up
    rows) and ``w_down [E, D, F]``.  The shared expert has the same form; with ``shared_gate``
    its result is multiplied by ``sigmoid(w_sg x)``, one number per token.

    Few rows (and every single-token step, so that a recorded step never asks the host): in
    bfloat16 the pairs are put in the order of their experts on the device and one kernel per
    product reads each expert's matrix once for all of its rows (matrix cores); in float32, and
    for sizes that kernel does not take, kernels that take one (token, expert) pair at a time.
    More rows: the pairs are put in the
    order of their experts on the device and the host reads where each expert's rows begin;
    shares of similar size are padded to the largest and all experts are ONE batched product,
    else each expert's rows are one product (the matrix library for bfloat16, the library's own
    float32 kernels otherwise); a last kernel adds every token's pairs in the order of its
    choice, so the result does not depend on what else the step holds."""

    libraries = ("routed_experts",)
    replayable = True          # single-token steps read nothing on the host

    def __init__(self, spec: RoutedExpertsSpec, runtime: Runtime):
        if spec.activation not in RE.EXPERT_ACTIVATIONS:
            raise ValueError(f"activation '{spec.activation}': {RE.EXPERT_ACTIVATIONS}")
        if spec.n_experts % spec.n_groups or not 1 <= spec.keep_groups <= spec.n_groups or \
                not 1 <= spec.top <= spec.keep_groups * (spec.n_experts // spec.n_groups):
            raise ValueError(f"routed experts: top {spec.top} of {spec.n_experts} experts in "
                             f"{spec.n_groups} groups of which {spec.keep_groups} are kept")
        self.spec = spec
        self.rt = runtime
        if spec.scoring not in RE.ROUTER_SCORINGS or not 1 <= spec.group_top <= RE.MAX_GROUP_TOP:
            raise ValueError(f"routed experts: scoring '{spec.scoring}' ({sorted(RE.ROUTER_SCORINGS)}), "
                             f"group_top {spec.group_top} (1..{RE.MAX_GROUP_TOP})")
        if spec.gated and spec.activation not in K.GATE_ACTIVATIONS:
            raise ValueError(f"gated experts: activation '{spec.activation}': {sorted(K.GATE_ACTIVATIONS)}")
        self.up_rows = (2 if spec.gated else 1) * spec.hidden
        self.w_router = self.w_up = self.w_down = self.shared_up = self.shared_down = None
        self.correction = self.shared_gate = None
        self.last_chosen = None

    def parameters(self):
        s = self.spec
        p = {"w_router": Param((s.n_experts, s.dim)),
             "w_up": Param((s.n_experts, self.up_rows, s.dim)),
             "w_down": Param((s.n_experts, s.dim, s.hidden))}
        if s.choice_correction:
            p["correction"] = Param((s.n_experts,), role="vector", init="around_zero")
        if s.shared_hidden:
            p["shared_up"] = Param(((2 if s.gated else 1) * s.shared_hidden, s.dim))
            p["shared_down"] = Param((s.dim, s.shared_hidden))
            if s.shared_gate:
                p["shared_gate"] = Param((1, s.dim))
        return p

    def bind(self, tensors):
        check_bound("RoutedExperts", self.parameters(), tensors)
        # zero rows up to a multiple of eight: the products' kernels store whole groups
        self.w_router = L.pad_rows(tensors["w_router"], 8)
        self.w_up, self.w_down = tensors["w_up"], tensors["w_down"]
        self.shared_up, self.shared_down = tensors.get("shared_up"), tensors.get("shared_down")
        if "correction" in tensors:
            self.correction = tensors["correction"].to(torch.float32).contiguous()
        if "shared_gate" in tensors:
            # one more row of the router's matrix: the gate's sum comes with the logits
            self.shared_gate = True
            self.w_router = L.pad_rows(torch.cat([tensors["w_router"], tensors["shared_gate"]], 0), 8)

    def step_flops(self, q_lens, starts) -> float:
        s = self.spec
        mats = 3 if s.gated else 2
        per_token = s.n_experts * s.dim + mats * s.top * s.hidden * s.dim + mats * s.shared_hidden * s.dim
        return 2.0 * sum(q_lens) * per_token

    def unread_bytes(self, rows: int) -> int:
        """The experts that the last step of ``rows`` tokens did not choose (read from the
        device: not for a timed region); before any such step, the ``E (1 - top / E)^rows``
        that a router which spreads its choices evenly leaves unread on average."""
        s = self.spec
        last = self.last_chosen
        if last is not None and last.shape[0] == rows:
            idle = s.n_experts - int(torch.unique(last).numel())
        else:
            idle = int(s.n_experts * (1.0 - s.top / s.n_experts) ** rows)
        per_expert = (self.w_up[0].numel() + self.w_down[0].numel()) * self.w_up.element_size()
        return idle * per_expert

    def _routed(self, x, chosen, weights, y, batch):
        s = self.spec
        n = x.shape[0]
        few = n <= PAIRWISE_MAX_ROWS or getattr(batch, "is_decode", False)
        if few and n >= GROUPED_MIN_ROWS and RE.grouped_rows_take(x, self.w_up) and s.hidden % 8 == 0:
            offsets, order, place = RE.expert_order(chosen, s.n_experts)
            if s.gated:
                # the float32 sums of the gate rows and the up rows, then the gate
                sums = RE.grouped_rows(x, order, s.top, self.w_up, offsets, None, n)
                h = K.gate_mul_sums(sums, s.activation)
            else:
                h = RE.grouped_rows(x, order, s.top, self.w_up, offsets, s.activation, n)
            ys = RE.grouped_rows(h, None, 1, self.w_down, offsets, None, n)
            return RE.combine_pairs(ys, place, weights, out=y)
        if few:
            return RE.experts_few_rows(x, self.w_up, self.w_down, chosen, weights, s.activation, out=y,
                                       gated=s.gated)
        offsets, order, place = RE.expert_order(chosen, s.n_experts)
        bounds = offsets.cpu().tolist()                         # the host learns the experts' shares
        most = max(bounds[e + 1] - bounds[e] for e in range(s.n_experts))
        cap = (most + PAD_ROWS_TO - 1) // PAD_ROWS_TO * PAD_ROWS_TO
        if s.n_experts * cap <= PADDED_MAX_WASTE * n * s.top:
            # shares of similar size: each padded to the largest, one batched product for all
            xs = RE.gather_pairs_padded(x, order, offsets, s.top, s.n_experts, cap)
            hs = torch.empty((s.n_experts, cap, self.up_rows), dtype=x.dtype, device=x.device)
            self._batched(xs, self.w_up, hs)
            hs = self._activated(hs.view(-1, self.up_rows)).view(s.n_experts, cap, s.hidden)
            ys = torch.empty((s.n_experts, cap, s.dim), dtype=x.dtype, device=x.device)
            self._batched(hs, self.w_down, ys)
            return RE.combine_pairs(ys.view(-1, s.dim), RE.padded_places(place, chosen, offsets, cap),
                                    weights, out=y)
        xs = RE.gather_pairs(x, order, s.top)
        hs = torch.empty((xs.shape[0], self.up_rows), dtype=x.dtype, device=x.device)
        ys = torch.empty((xs.shape[0], s.dim), dtype=x.dtype, device=x.device)
        for e in range(s.n_experts):
            a, b = bounds[e], bounds[e + 1]
            if b > a:
                self._product(xs[a:b], self.w_up[e], hs[a:b])
        hs = self._activated(hs)
        for e in range(s.n_experts):
            a, b = bounds[e], bounds[e + 1]
            if b > a:
                self._product(hs[a:b], self.w_down[e], ys[a:b])
        return RE.combine_pairs(ys, place, weights, out=y)

    def _activated(self, h):
        """The inner rows from the first product's rows [P, F] (or [P, 2 F]: gate, then up)."""
        if self.spec.gated:
            return K.gate_mul(h, self.spec.activation)
        return K.activate(h, self.spec.activation, out=h)

    def _batched(self, a, w, out):
        """out[e] = a[e] w[e]^T for every expert: a [E, cap, K], w [E, M, K], out [E, cap, M]."""
        if a.dtype == torch.float32:
            return K.gemm_f32_batched(a, w, out)
        return torch.bmm(a, w.transpose(1, 2), out=out)         # the vendor library, as for prompts

    def _product(self, a, w, out):
        if a.dtype == torch.float32:
            return K.gemm_f32(a, w, out=out)
        return torch.matmul(a, w.t(), out=out)                  # the vendor library, as for prompts

    def forward_rows(self, x, batch):
        """The feed-forward's output alone, float32 [N, D]."""
        s = self.spec
        z = L.linear(x, self.w_router, out_dtype=torch.float32)
        chosen, weights = RE.route(z, s.n_experts, s.top, s.n_groups, s.keep_groups, s.weight_eps,
                                   scoring=s.scoring, correction=self.correction, group_top=s.group_top)
        self.last_chosen = chosen                  # a replayed step leaves its choice here as well
        y = None
        if s.shared_hidden:
            if s.gated:
                h = L.gated_linear(x, self.shared_up, s.activation)
            else:
                h = L.linear(x, self.shared_up)
                K.activate(h, s.activation, out=h)
            y = L.linear(h, self.shared_down, out_dtype=torch.float32)
            if self.shared_gate:
                K.scale_rows_sigmoid(y, z[:, s.n_experts:])
        return self._routed(x, chosen, weights, y, batch)

    def forward(self, x, batch, residual):
        K.add_into(residual, self.forward_rows(x, batch))


register_feed_forward("routed_experts", RoutedExperts)
