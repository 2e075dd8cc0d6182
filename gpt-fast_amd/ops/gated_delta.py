"""Python faces of the gated-delta-rule kernels of csrc/gated_delta.hip: the short causal
convolutions with their tails, and the cell token by token.  Shape checks on the host, then
the launch."""
import ctypes
from dataclasses import dataclass

import torch

from .library import KernelError, check, library, ptr, require_contiguous, require_device, stream_handle

_i, _f, _sz = ctypes.c_int, ctypes.c_float, ctypes.c_size_t

MAX_KEY_DIM = 512            # rows of S a workgroup's threads hold in registers
MAX_TAPS = 16


@dataclass(frozen=True)
class RowLayout:
    """Where a token's values lie in a row of the fused projection (column offsets, in
    elements): the convolved channels q, k, v first (``conv`` of them), then the
    pre-activations of beta and of the decay (one per head each), then the output gate."""
    width: int
    conv: int
    b: int
    a: int
    g: int

    @staticmethod
    def fused(n_heads: int, n_kv_heads: int, key_dim: int, value_dim: int) -> "RowLayout":
        conv = 2 * n_kv_heads * key_dim + n_heads * value_dim
        b = conv
        a = b + n_heads
        g = a + n_heads
        return RowLayout(g + n_heads * value_dim, conv, b, a, g)


def state_size(n_heads: int, n_kv_heads: int, key_dim: int, value_dim: int, taps: int) -> int:
    """float32 elements of one sequence's state: S [H, dk, dv], then the convolutions' last
    ``taps - 1`` inputs [taps - 1, C]."""
    conv = 2 * n_kv_heads * key_dim + n_heads * value_dim
    return n_heads * key_dim * value_dim + (taps - 1) * conv


def _check_step(proj, layout, state, q_start, slots, n_seqs):
    for name, t in (("proj", proj), ("state", state)):
        if t.dtype != torch.float32:
            raise KernelError(f"gated delta: {name} must be float32, is {t.dtype}")
    for name, t in (("q_start", q_start), ("slots", slots)):
        if t.dtype != torch.int32:
            raise KernelError(f"gated delta: {name} must be int32")
    if proj.dim() != 2 or proj.shape[1] != layout.width:
        raise KernelError(f"gated delta: rows are {tuple(proj.shape)}, expected [N, {layout.width}]")
    if q_start.numel() < n_seqs + 1 or slots.numel() < n_seqs:
        raise KernelError("gated delta: q_start / slots are shorter than the batch")


def short_conv(proj: torch.Tensor, layout: RowLayout, taps: torch.Tensor, state: torch.Tensor,
               tail_offset: int, tok_seq, q_start, slots, n_seqs: int) -> torch.Tensor:
    """silu of the causal convolution of the first ``layout.conv`` columns of proj over each
    sequence's tokens, float32 [N, C]; taps float32 [C, K], the last column the current
    token's.  ``state`` [slots, size] holds every sequence's last K - 1 inputs at
    ``tail_offset`` ([K - 1, C], oldest first; zero for a new sequence) and is left holding the
    step's."""
    require_device(proj, taps, state, tok_seq, q_start, slots)
    require_contiguous(proj=proj, taps=taps, state=state, tok_seq=tok_seq, q_start=q_start, slots=slots)
    _check_step(proj, layout, state, q_start, slots, n_seqs)
    C = layout.conv
    if taps.dtype != torch.float32 or taps.dim() != 2 or taps.shape[0] != C or not 1 <= taps.shape[1] <= MAX_TAPS:
        raise KernelError(f"short_conv: taps must be float32 [{C}, 1..{MAX_TAPS}]")
    K = taps.shape[1]
    if state.dim() != 2 or tail_offset < 0 or tail_offset + (K - 1) * C > state.shape[1]:
        raise KernelError("short_conv: the tails do not fit the state")
    if tok_seq.dtype != torch.int32 or tok_seq.numel() < proj.shape[0]:
        raise KernelError("short_conv: tok_seq must be int32 and cover the batch")
    y = torch.empty((proj.shape[0], C), dtype=torch.float32, device=proj.device)
    check(library("gated_delta").gfa_short_conv(
        ptr(proj), _i(layout.width), ptr(taps), _i(K), _i(C), ptr(state), _sz(state.stride(0)),
        _sz(tail_offset), ptr(tok_seq), ptr(q_start), ptr(slots), ptr(y), _i(proj.shape[0]),
        _i(n_seqs), stream_handle()), "short_conv")
    return y


CHUNKS_FROM_TOKENS = 16      # runs shorter than this go token by token


def chunks_available(key_dim: int, value_dim: int) -> bool:
    return bool(library("gated_delta").gfa_gated_delta_chunks_take(_i(key_dim), _i(value_dim)))


def cell(conv, proj, layout, A_log, dt_bias, state, q_start, slots, n_seqs, max_q_len, n_heads,
         n_kv_heads, key_dim, value_dim, q_scale, unit_eps) -> torch.Tensor:
    """Which kernel runs the cell: token by token for short runs (single-token steps), a chunk
    of tokens at a time where some sequence brings many."""
    chunked = max_q_len >= CHUNKS_FROM_TOKENS and chunks_available(key_dim, value_dim)
    return scan(conv, proj, layout, A_log, dt_bias, state, q_start, slots, n_seqs, n_heads, n_kv_heads,
                key_dim, value_dim, q_scale, unit_eps, chunked=chunked, max_q_len=max_q_len)


def scan(conv: torch.Tensor, proj: torch.Tensor, layout: RowLayout, A_log: torch.Tensor,
         dt_bias: torch.Tensor, state: torch.Tensor, q_start, slots, n_seqs: int, n_heads: int,
         n_kv_heads: int, key_dim: int, value_dim: int, q_scale: float, unit_eps: float,
         chunked: bool = False, max_q_len: int = 64) -> torch.Tensor:
    """The cell over every sequence's new tokens in order; ``state`` [slots, size] holds S
    [H, dk, dv] at its start and is read and left updated.  conv float32 [N, C]: q, k, v after
    their convolutions; proj float32 [N, layout.width] holds the pre-activations of beta and
    of the decay; A_log, dt_bias float32 [H].  Returns o float32 [N, H * dv].  ``chunked``:
    the kernel that takes a chunk of tokens at a time (the same arithmetic written out; chunks
    of 64 tokens if ``max_q_len``, the longest run of new tokens, is beyond 32, else of 32)."""
    require_device(conv, proj, A_log, dt_bias, state, q_start, slots)
    require_contiguous(conv=conv, proj=proj, A_log=A_log, dt_bias=dt_bias, state=state,
                       q_start=q_start, slots=slots)
    _check_step(proj, layout, state, q_start, slots, n_seqs)
    C = 2 * n_kv_heads * key_dim + n_heads * value_dim
    if conv.dtype != torch.float32 or tuple(conv.shape) != (proj.shape[0], C) or layout.conv != C:
        raise KernelError(f"gated delta: the convolved rows must be float32 [N, {C}]")
    for name, t in (("A_log", A_log), ("dt_bias", dt_bias)):
        if t.dtype != torch.float32 or t.numel() != n_heads:
            raise KernelError(f"gated delta: {name} must be float32 [{n_heads}]")
    if n_heads % n_kv_heads or key_dim > MAX_KEY_DIM:
        raise KernelError(f"gated delta: {n_heads} heads over {n_kv_heads} key heads of {key_dim}")
    if state.dim() != 2 or state.shape[1] < n_heads * key_dim * value_dim:
        raise KernelError("gated delta: the state is smaller than S [H, dk, dv]")
    out = torch.empty((proj.shape[0], n_heads * value_dim), dtype=torch.float32, device=proj.device)
    lib = library("gated_delta")
    if chunked and not chunks_available(key_dim, value_dim):
        raise KernelError("gated delta: the chunked kernel does not take these sizes")
    head = (ptr(conv), _i(C), ptr(proj), _i(layout.width), _i(layout.b), _i(layout.a), ptr(A_log),
            ptr(dt_bias), ptr(state), _sz(state.stride(0)), ptr(q_start), ptr(slots), ptr(out), _i(n_seqs))
    tail = (_i(n_heads), _i(n_kv_heads), _i(key_dim), _i(value_dim), _f(q_scale), _f(unit_eps),
            stream_handle())
    if chunked:
        check(lib.gfa_gated_delta_chunks(*head, _i(int(max_q_len)), *tail), "gated_delta_chunks")
    else:
        check(lib.gfa_gated_delta_scan(*head, *tail), "gated_delta_scan")
    return out
