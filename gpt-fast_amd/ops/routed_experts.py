"""Python faces of csrc/routed_experts.hip: the router's choice per token and the products of
the chosen experts.  Shape checks on the host, then the launch."""
import ctypes
from typing import Optional

import torch

from .kernels import ACTIVATIONS
from .library import KernelError, check, library, ptr, require_contiguous, require_device, stream_handle

_i, _f, _ll = ctypes.c_int, ctypes.c_float, ctypes.c_longlong
EXPERT_ACTIVATIONS = ("silu", "gelu_tanh", "gelu")
MAX_EXPERTS = 1024
MAX_TOP = 64
# steps of up to this many tokens take the form of grouped_rows in which every wave reads its
# own pieces of x (no barriers); more tokens share x through LDS
DIRECT_X_MAX_ROWS = 4


def _is_bf16(t: torch.Tensor) -> int:
    if t.dtype == torch.bfloat16:
        return 1
    if t.dtype == torch.float32:
        return 0
    raise KernelError(f"activation dtype {t.dtype}: float32 or bfloat16 only")


ROUTER_SCORINGS = {"softmax": 0, "sigmoid": 1}
MAX_GROUP_TOP = 8


def route(z: torch.Tensor, n_experts: int, top: int, groups: int, keep: int, weight_eps: float,
          scoring: str = "softmax", correction: Optional[torch.Tensor] = None, group_top: int = 1):
    """(chosen int32 [N, top], weights float32 [N, top]) from router logits z float32
    [N, >= n_experts] (a view of wider rows is allowed): scores s = softmax over the experts, or
    sigmoid of each (``scoring``); the choice is made on s + ``correction`` (float32
    [n_experts]; None: on s): the ``keep`` best of ``groups`` equal groups of neighbours by the
    sum of their ``group_top`` largest choice scores (1: by their largest), of their experts
    the ``top`` with the largest choice scores in falling order; each weighted by its s over
    the chosen experts' s summed, plus ``weight_eps``."""
    require_device(z, correction)
    require_contiguous(correction=correction)
    if z.dtype != torch.float32 or z.dim() != 2 or z.shape[1] < n_experts or z.stride(1) != 1:
        raise KernelError(f"route: z must be float32 [N, >= {n_experts}] with unit stride along a row")
    if not (0 < n_experts <= MAX_EXPERTS and groups > 0 and n_experts % groups == 0
            and 1 <= keep <= groups and 1 <= top <= min(MAX_TOP, keep * (n_experts // groups))):
        raise KernelError(f"route: {n_experts} experts, top {top}, {keep} of {groups} groups: "
                          f"not a choice this kernel makes")
    if scoring not in ROUTER_SCORINGS or not 1 <= group_top <= MAX_GROUP_TOP:
        raise KernelError(f"route: scoring '{scoring}' ({sorted(ROUTER_SCORINGS)}), group_top {group_top} "
                          f"(1..{MAX_GROUP_TOP})")
    if correction is not None and (correction.dtype != torch.float32 or correction.numel() != n_experts):
        raise KernelError(f"route: correction must be float32 [{n_experts}]")
    n = z.shape[0]
    chosen = torch.empty((n, top), dtype=torch.int32, device=z.device)
    weights = torch.empty((n, top), dtype=torch.float32, device=z.device)
    check(library("routed_experts").gfa_route(ptr(z), _ll(z.stride(0)), _i(n), _i(n_experts), _i(top),
                                              _i(groups), _i(keep), _f(weight_eps),
                                              _i(ROUTER_SCORINGS[scoring]), ptr(correction), _i(group_top),
                                              ptr(chosen), ptr(weights), stream_handle()), "route")
    return chosen, weights


def _check_experts(x, w_up, w_down, chosen, weights, gated=False):
    require_device(x, w_up, w_down, chosen, weights)
    require_contiguous(x=x, w_up=w_up, w_down=w_down, chosen=chosen, weights=weights)
    inner = w_up.shape[1] // 2 if gated and w_up.dim() == 3 else (w_up.shape[1] if w_up.dim() == 3 else -1)
    if w_up.dim() != 3 or w_down.dim() != 3 or w_up.shape[0] != w_down.shape[0] or \
            w_up.shape[2] != x.shape[1] or tuple(w_down.shape[1:]) != (w_up.shape[2], inner) or \
            (gated and w_up.shape[1] % 2):
        raise KernelError(f"experts: w_up {tuple(w_up.shape)} must be [E, F, D] ([E, 2 F, D] for gated "
                          f"experts) and w_down {tuple(w_down.shape)} [E, D, F] for x {tuple(x.shape)}")
    if w_up.dtype != x.dtype or w_down.dtype != x.dtype:
        raise KernelError("experts: x and the weights must have one type")
    if chosen.dtype != torch.int32 or weights.dtype != torch.float32 or chosen.shape != weights.shape \
            or chosen.dim() != 2 or chosen.shape[0] != x.shape[0]:
        raise KernelError("experts: chosen int32 and weights float32 must both be [N, top]")


def experts_few_rows(x: torch.Tensor, w_up: torch.Tensor, w_down: torch.Tensor, chosen: torch.Tensor,
                     weights: torch.Tensor, activation: str, out: Optional[torch.Tensor] = None,
                     gated: bool = False):
    """float32 [N, D] (+)= sum_k weights[n, k] W_down[e] act(W_up[e] x_n), e = chosen[n, k]: one
    (token, expert) pair at a time, each weight row read once per pair.  ``gated``: W_up is
    [E, 2 F, D], an expert's F gate rows and then its F up rows, and the inner row is
    act(W_gate[e] x) * (W_up[e] x).  ``out``: the sums are added to it."""
    _check_experts(x, w_up, w_down, chosen, weights, gated)
    if activation not in EXPERT_ACTIVATIONS:
        raise KernelError(f"experts: activation '{activation}': {EXPERT_ACTIVATIONS}")
    n, D = x.shape
    F, top = w_down.shape[2], chosen.shape[1]
    if n * top > 65535 or D * 4 > 65536 or top * F * 4 > 65536:
        raise KernelError("experts_few_rows: too many pairs or too long rows for this kernel")
    accumulate = out is not None
    if out is None:
        out = torch.empty((n, D), dtype=torch.float32, device=x.device)
    elif tuple(out.shape) != (n, D) or out.dtype != torch.float32 or not out.is_contiguous():
        raise KernelError("experts_few_rows: out must be contiguous float32 [N, D]")
    h = torch.empty((n * top, F), dtype=x.dtype, device=x.device)
    check(library("routed_experts").gfa_experts_few_rows(
        ptr(x), ptr(w_up), ptr(w_down), ptr(chosen), ptr(weights), ptr(h), ptr(out), _i(n), _i(top),
        _i(D), _i(F), _i(ACTIVATIONS[activation]), _i(int(bool(gated))), _i(int(accumulate)),
        _i(_is_bf16(x)), stream_handle()), "experts_few_rows")
    return out


def expert_order(chosen: torch.Tensor, n_experts: int):
    """(offsets int32 [E + 1], order int32 [P], place int32 [P]) for the P = N top pairs of
    ``chosen``: the pairs in the order of their experts (``order[i]`` = the pair at place i,
    ``place[p]`` = where pair p went), expert e's pairs at places offsets[e] .. offsets[e+1]-1."""
    require_device(chosen)
    require_contiguous(chosen=chosen)
    if chosen.dtype != torch.int32:
        raise KernelError("expert_order: chosen must be int32")
    P = chosen.numel()
    offsets = torch.empty(n_experts + 1, dtype=torch.int32, device=chosen.device)
    order = torch.empty(P, dtype=torch.int32, device=chosen.device)
    place = torch.empty(P, dtype=torch.int32, device=chosen.device)
    check(library("routed_experts").gfa_expert_order(ptr(chosen), _i(P), _i(n_experts), ptr(offsets),
                                                     ptr(order), ptr(place), stream_handle()),
          "expert_order")
    return offsets, order, place


def gather_pairs(x: torch.Tensor, order: torch.Tensor, top: int) -> torch.Tensor:
    """[P, D]: row i is x[order[i] // top]."""
    require_device(x, order)
    require_contiguous(x=x, order=order)
    out = torch.empty((order.numel(), x.shape[1]), dtype=x.dtype, device=x.device)
    check(library("routed_experts").gfa_gather_pairs(ptr(x), ptr(order), ptr(out), _i(order.numel()),
                                                     _i(top), _i(x.shape[1]), _i(_is_bf16(x)),
                                                     stream_handle()), "gather_pairs")
    return out


def gather_pairs_padded(x: torch.Tensor, order: torch.Tensor, offsets: torch.Tensor, top: int,
                        n_experts: int, cap: int) -> torch.Tensor:
    """[E, cap, D]: expert e's rows ``x[order[offsets[e] + i] // top]`` for i below its count,
    zero rows beyond; ``cap`` must be at least the largest count (the caller's to know)."""
    require_device(x, order, offsets)
    require_contiguous(x=x, order=order, offsets=offsets)
    if offsets.dtype != torch.int32 or offsets.numel() != n_experts + 1 or order.dtype != torch.int32 \
            or cap < 1 or x.dim() != 2:
        raise KernelError("gather_pairs_padded: offsets int32 [E + 1], order int32, cap >= 1")
    out = torch.empty((n_experts, cap, x.shape[1]), dtype=x.dtype, device=x.device)
    check(library("routed_experts").gfa_gather_pairs_padded(
        ptr(x), ptr(order), ptr(offsets), ptr(out), _i(n_experts), _i(cap), _i(top), _i(x.shape[1]),
        _i(_is_bf16(x)), stream_handle()), "gather_pairs_padded")
    return out


def padded_places(place: torch.Tensor, chosen: torch.Tensor, offsets: torch.Tensor, cap: int) -> torch.Tensor:
    """int32 [P]: the row of pair p in the [E * cap] rows of :func:`gather_pairs_padded`."""
    require_device(place, chosen, offsets)
    require_contiguous(place=place, chosen=chosen, offsets=offsets)
    if place.dtype != torch.int32 or chosen.dtype != torch.int32 or offsets.dtype != torch.int32 \
            or place.numel() != chosen.numel():
        raise KernelError("padded_places: place, chosen [P] and offsets must be int32")
    out = torch.empty(place.numel(), dtype=torch.int32, device=place.device)
    check(library("routed_experts").gfa_padded_places(ptr(place), ptr(chosen), ptr(offsets), ptr(out),
                                                      _i(place.numel()), _i(cap), stream_handle()),
          "padded_places")
    return out


def combine_pairs(ys: torch.Tensor, place: torch.Tensor, weights: torch.Tensor,
                  out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """float32 [N, D] (+)= sum_k weights[n, k] ys[place[n top + k]], in the order of k; every
    place must be a row of ys (the caller's to know)."""
    require_device(ys, place, weights, out)
    require_contiguous(ys=ys, place=place, weights=weights, out=out)
    n, top = weights.shape
    D = ys.shape[1]
    if ys.shape[0] < n * top or place.numel() != n * top or weights.dtype != torch.float32:
        raise KernelError("combine_pairs: ys [>= N top, D], place [N top] and weights [N, top] do not fit")
    accumulate = out is not None
    if out is None:
        out = torch.empty((n, D), dtype=torch.float32, device=ys.device)
    elif tuple(out.shape) != (n, D) or out.dtype != torch.float32:
        raise KernelError("combine_pairs: out must be float32 [N, D]")
    check(library("routed_experts").gfa_combine_pairs(ptr(ys), ptr(place), ptr(weights), ptr(out), _i(n),
                                                      _i(top), _i(D), _i(int(accumulate)),
                                                      _i(_is_bf16(ys)), stream_handle()), "combine_pairs")
    return out


def grouped_rows_take(x: torch.Tensor, w: torch.Tensor) -> bool:
    """Whether :func:`grouped_rows` takes these operands: bfloat16, rows of a multiple of eight
    elements at addresses that are multiples of 16."""
    return (x.dtype == torch.bfloat16 and w.dtype == torch.bfloat16 and x.dim() == 2 and w.dim() == 3
            and x.shape[1] == w.shape[2] and x.shape[1] % 8 == 0 and x.is_contiguous()
            and w.is_contiguous() and x.data_ptr() % 16 == 0 and w.data_ptr() % 16 == 0)


def grouped_rows(x: torch.Tensor, order: Optional[torch.Tensor], top: int, w: torch.Tensor,
                 offsets: torch.Tensor, activation: Optional[str], rows_at_most: int) -> torch.Tensor:
    """[P, N]: row ``offsets[e] + i`` is ``W[e] x[r]`` for expert e's i-th pair, r = the pair's
    token ``order[.] // top`` (or, without ``order``, the row at the same place of x, which then
    has P rows).  With an activation the result is act(.) in bfloat16, else the float32 sums.
    x bfloat16 [rows, K], W bfloat16 [E, N, K], offsets int32 [E + 1] as :func:`expert_order`
    gives them; ``rows_at_most``: the most pairs one expert can have.  One pass over each
    expert's matrix whatever the number of its rows; nothing is read on the host."""
    require_device(x, order, w, offsets)
    require_contiguous(x=x, order=order, w=w, offsets=offsets)
    if not grouped_rows_take(x, w):
        raise KernelError("grouped_rows: bfloat16 x [rows, K] and W [E, N, K] with K a multiple of 8")
    E, N, K = w.shape
    if offsets.dtype != torch.int32 or offsets.numel() != E + 1:
        raise KernelError(f"grouped_rows: offsets must be int32 [{E + 1}]")
    if order is not None:
        if order.dtype != torch.int32 or top < 1 or order.numel() > x.shape[0] * top:
            raise KernelError("grouped_rows: order must be int32 with at most rows * top elements")
        P = order.numel()
    else:
        P, top = x.shape[0], 1
    if activation is not None and activation not in EXPERT_ACTIVATIONS:
        raise KernelError(f"grouped_rows: activation '{activation}': {EXPERT_ACTIVATIONS}")
    out = torch.empty((P, N), dtype=torch.float32 if activation is None else torch.bfloat16,
                      device=x.device)
    check(library("routed_experts").gfa_grouped_rows(
        ptr(x), ptr(order), _i(top), ptr(w), ptr(offsets), ptr(out), _i(E), _i(N), _i(K),
        _i(-1 if activation is None else ACTIVATIONS[activation]), _i(max(1, int(rows_at_most))),
        _i(int(rows_at_most <= DIRECT_X_MAX_ROWS)), stream_handle()), "grouped_rows")
    return out
