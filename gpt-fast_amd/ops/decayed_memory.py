"""Python faces of the decayed-memory (lightning attention) kernels of csrc/decayed_memory.hip:
shape checks on the host, then the launch."""
import ctypes
from dataclasses import dataclass
from typing import Optional

import torch

from .library import KernelError, check, library, ptr, require_contiguous, require_device, stream_handle

_i, _f, _sz = ctypes.c_int, ctypes.c_float, ctypes.c_size_t

MAX_KEY_DIM = 512            # rows of S a workgroup's threads hold in registers


@dataclass(frozen=True)
class RowLayout:
    """Where a token's q, k, v and output gate lie in a row of the fused projection (column
    offsets, in elements)."""
    width: int
    q: int
    k: int
    v: int
    g: int

    @staticmethod
    def fused(n_heads: int, key_dim: int, value_dim: int) -> "RowLayout":
        """Rows of q, k, v, g one after the other."""
        k = n_heads * key_dim
        v = k + n_heads * key_dim
        g = v + n_heads * value_dim
        return RowLayout(g + n_heads * value_dim, 0, k, v, g)


def state_size(n_heads: int, key_dim: int, value_dim: int) -> int:
    """float32 elements of one sequence's state: S [H, dk, dv]."""
    return n_heads * key_dim * value_dim


CHUNKS_FROM_TOKENS = 32      # runs shorter than this go token by token


def cell(proj, layout, decay, state, q_start, slots, n_seqs, max_q_len, n_heads, key_dim,
         value_dim, activation: bool = True) -> torch.Tensor:
    """Which kernel runs the cell: token by token for short runs (single-token steps), a
    chunk of tokens at a time where some sequence brings many."""
    chunked = max_q_len >= CHUNKS_FROM_TOKENS and chunks_available(key_dim, value_dim)
    return scan(proj, layout, decay, state, q_start, slots, n_seqs, n_heads, key_dim, value_dim,
                chunked=chunked, activation=activation)


def chunks_available(key_dim: int, value_dim: int) -> bool:
    lib = library("decayed_memory")
    return hasattr(lib, "gfa_decayed_memory_chunks") and bool(
        lib.gfa_decayed_memory_chunks_take(_i(key_dim), _i(value_dim)))


def scan(proj: torch.Tensor, layout: RowLayout, decay: torch.Tensor, state: torch.Tensor,
         q_start: torch.Tensor, slots: torch.Tensor, n_seqs: int, n_heads: int, key_dim: int,
         value_dim: int, chunked: bool = False, activation: bool = True) -> torch.Tensor:
    """The cell over every sequence's new tokens in order; ``state`` [slots, state_size] is
    read and left updated.  proj float32 [N, layout.width] holds the pre-activations of q, k
    and v (``activation`` False: q, k and v themselves); decay float32 [H]; returns o float32
    [N, H * dv]."""
    require_device(proj, decay, state, q_start, slots)
    require_contiguous(proj=proj, decay=decay, state=state, q_start=q_start, slots=slots)
    for name, t in (("proj", proj), ("decay", decay), ("state", state)):
        if t.dtype != torch.float32:
            raise KernelError(f"decayed memory: {name} must be float32, is {t.dtype}")
    for name, t in (("q_start", q_start), ("slots", slots)):
        if t.dtype != torch.int32:
            raise KernelError(f"decayed memory: {name} must be int32")
    if proj.dim() != 2 or proj.shape[1] != layout.width:
        raise KernelError(f"decayed memory: rows are {tuple(proj.shape)}, expected [N, {layout.width}]")
    if max(layout.q, layout.k) + n_heads * key_dim > layout.width or \
            layout.v + n_heads * value_dim > layout.width:
        raise KernelError("decayed memory: the row layout does not fit the row width")
    if decay.numel() != n_heads:
        raise KernelError("decayed memory: one decay per head")
    if state.dim() != 2 or state.shape[1] != state_size(n_heads, key_dim, value_dim):
        raise KernelError(f"decayed memory: state is {tuple(state.shape)}, expected "
                          f"[slots, {state_size(n_heads, key_dim, value_dim)}]")
    if q_start.numel() < n_seqs + 1 or slots.numel() < n_seqs:
        raise KernelError("decayed memory: q_start / slots are shorter than the batch")
    if key_dim > MAX_KEY_DIM:
        raise KernelError(f"decayed memory: key_dim {key_dim} > {MAX_KEY_DIM} is not supported")
    out = torch.empty((proj.shape[0], n_heads * value_dim), dtype=torch.float32, device=proj.device)
    args = (ptr(proj), ptr(decay), ptr(state), _sz(state.stride(0)), ptr(q_start), ptr(slots),
            ptr(out), _i(n_seqs), _i(n_heads), _i(key_dim), _i(value_dim), _i(layout.width),
            _i(layout.q), _i(layout.k), _i(layout.v), _i(int(bool(activation))))
    lib = library("decayed_memory")
    if chunked:
        if not chunks_available(key_dim, value_dim):
            raise KernelError("decayed memory: the chunked kernel does not take these sizes")
        check(lib.gfa_decayed_memory_chunks(*args, stream_handle()), "decayed_memory_chunks")
    else:
        check(lib.gfa_decayed_memory_scan(*args, stream_handle()), "decayed_memory_scan")
    return out


def row_norm_gate(o: torch.Tensor, weight: Optional[torch.Tensor], proj: torch.Tensor, layout: RowLayout,
                  eps: float, out_dtype: torch.dtype, groups: int = 1, gate: str = "sigmoid") -> torch.Tensor:
    """y[t, :] = o[t, :] / rms(o[t, :]) * weight * gate(g[t, :]) in ``out_dtype``, the root mean
    square taken over each of ``groups`` equal parts of the row (1: the whole row; the number
    of heads: every head by itself); o float32 [N, W]; ``weight`` float32 of W elements, or of
    fewer that divide W and are used again along the row (one weight shared by the heads), or
    None; the gate's pre-activations lie in proj at ``layout.g``; ``gate`` "sigmoid" or
    "silu"."""
    require_device(o, weight, proj)
    require_contiguous(o=o, weight=weight, proj=proj)
    n, width = o.shape
    if o.dtype != torch.float32 or groups < 1 or width % groups:
        raise KernelError("row_norm_gate: o must be float32 with rows that divide into the groups")
    if weight is not None and (weight.dtype != torch.float32 or weight.numel() < 1
                               or width % weight.numel()):
        raise KernelError("row_norm_gate: weight must be float32 of a size that divides the row's width")
    if proj.dtype != torch.float32 or proj.shape != (n, layout.width) or layout.g + width > layout.width:
        raise KernelError("row_norm_gate: the projection's rows do not fit")
    if out_dtype not in (torch.float32, torch.bfloat16):
        raise KernelError(f"row_norm_gate: output type {out_dtype}")
    if gate not in ("sigmoid", "silu"):
        raise KernelError(f"row_norm_gate: gate '{gate}': sigmoid or silu")
    y = torch.empty((n, width), dtype=out_dtype, device=o.device)
    check(library("decayed_memory").gfa_row_norm_gate(
        ptr(o), ptr(weight), _i(0 if weight is None else weight.numel()), ptr(proj), _i(layout.width),
        _i(layout.g), ptr(y), _i(int(out_dtype == torch.bfloat16)), _i(n), _i(width), _i(groups),
        _i(int(gate == "silu")), _f(eps), stream_handle()), "row_norm_gate")
    return y
