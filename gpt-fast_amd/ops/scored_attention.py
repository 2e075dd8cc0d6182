"""Python faces of csrc/scored_attention.hip: attention over the paged cache with steps between
the dot product and the softmax (a temperature per head, a soft cap, a bias by distance, a mix
across heads), keys and values of different sizes, and the kernels that prepare q, keys and
values of the two mixers that use it.  Shape checks on the host, then the launch."""
import ctypes
import math
from typing import Optional

import torch

from .kernels import PAGE
from .library import KernelError, check, library, ptr, require_contiguous, require_device, stream_handle

_i, _f, _ll = ctypes.c_int, ctypes.c_float, ctypes.c_longlong


def _is_bf16(t: torch.Tensor) -> int:
    if t.dtype == torch.bfloat16:
        return 1
    if t.dtype == torch.float32:
        return 0
    raise KernelError(f"activation dtype {t.dtype}: float32 or bfloat16 only")


def _check_pages(k_pages, v_pages, G, hd, vd, dtype):
    for name, p, tail in (("k_pages", k_pages, (G, PAGE, hd)), ("v_pages", v_pages, (G, vd, PAGE))):
        if p is None:
            continue
        if p.dim() != 4 or tuple(p.shape[1:]) != tail:
            raise KernelError(f"{name} must be [n_pages, {tail[0]}, {tail[1]}, {tail[2]}], is {tuple(p.shape)}")
        if p.dtype != dtype or not p.is_contiguous():
            raise KernelError(f"{name} must be contiguous {dtype}")


def distance_rows(rows: int, far: float) -> list:
    """Row of a distance table of ``rows`` rows for every distance 0 .. ceil(far): with
    ``half = rows // 2``, distance n < half has row n; further ones share rows in logarithmic
    steps, ``half + floor(ln(n / half) / ln(far / half) * (rows - half))``, at most the last
    row.  Distances beyond the list have the last row.  Worked out in double precision."""
    half = rows // 2
    out = []
    for n in range(int(math.ceil(far)) + 1):
        if n < half or half == 0:
            out.append(min(n, rows - 1))
            continue
        step = math.log(n / half) / math.log(far / half) * (rows - half) if far > half else rows
        out.append(min(rows - 1, half + int(math.floor(step))))
    return out


def attention(q: torch.Tensor, k_pages: torch.Tensor, v_pages: torch.Tensor, tok_seq, tok_pos, table,
              scale: float, *, window: int = 0, temperature: Optional[torch.Tensor] = None,
              softcap: float = 0.0, bias: Optional[torch.Tensor] = None,
              lookup: Optional[torch.Tensor] = None, talk: Optional[torch.Tensor] = None,
              log_bias=None, sink: bool = False,
              head_major: bool = False, out: Optional[torch.Tensor] = None, step=None) -> torch.Tensor:
    """Each token's heads attend to the keys of its sequence's pages.  q is [N, H, hd], or
    [H, N, hd] if ``head_major`` (the result then lies the same way); k_pages
    [pages, G, 64, hd], v_pages [pages, G, vd, 64]; temperature float32 [H]; bias float32
    [rows, H] with lookup int32 [distances] (see :func:`distance_rows`); talk float32 [H, H];
    log_bias = (r1, r2), float32 [H] each: ``r1[h] ln(1 + r2[h] (i - j))`` is taken off the
    score; sink: the softmax's denominator has one more term exp(0).
    Returns [N, H, vd] (or [H, N, vd]) in q's type.  ``out`` may be a view with unit stride
    in its last dimension.  ``step`` = (q_start int32 [B + 1], start_pos int32 [B], B, longest
    run of new tokens) describes the same tokens sequence by sequence; with it, bfloat16 rows
    of sizes the matrix-core kernel takes go there."""
    r1, r2 = log_bias if log_bias is not None else (None, None)
    require_device(q, k_pages, v_pages, tok_seq, tok_pos, table, temperature, bias, lookup, talk, out,
                   r1, r2)
    require_contiguous(tok_seq=tok_seq, tok_pos=tok_pos, table=table, temperature=temperature,
                       bias=bias, lookup=lookup, talk=talk, r1=r1, r2=r2)
    if q.dim() != 3 or q.stride(2) != 1:
        raise KernelError("scored attention: q must have three dimensions, the last with unit stride")
    n, H = (q.shape[1], q.shape[0]) if head_major else (q.shape[0], q.shape[1])
    hd = q.shape[2]
    G, vd = k_pages.shape[1], v_pages.shape[2]
    if H % G:
        raise KernelError(f"scored attention: {H} heads do not divide into {G} kv heads")
    _check_pages(k_pages, v_pages, G, hd, vd, q.dtype)
    for name, t in (("tok_seq", tok_seq), ("tok_pos", tok_pos), ("table", table)):
        if t.dtype != torch.int32:
            raise KernelError(f"scored attention: {name} must be int32")
    if tok_seq.numel() < n or tok_pos.numel() < n:
        raise KernelError("scored attention: token maps are shorter than the batch")
    if (r1 is None) != (r2 is None):
        raise KernelError("scored attention: the bias by log distance needs both r1 and r2")
    for name, t, count in (("temperature", temperature, H), ("talk", talk, H * H), ("r1", r1, H),
                           ("r2", r2, H)):
        if t is not None and (t.dtype != torch.float32 or t.numel() != count):
            raise KernelError(f"scored attention: {name} must be float32 with {count} elements")
    rows = 0
    if bias is not None:
        if bias.dtype != torch.float32 or bias.dim() != 2 or bias.shape[1] != H or bias.shape[0] < 1:
            raise KernelError("scored attention: bias must be float32 [rows, H]")
        if lookup is None or lookup.dtype != torch.int32:
            raise KernelError("scored attention: a bias needs its int32 lookup table")
        rows = bias.shape[0]
    if talk is not None and H > 64:
        raise KernelError("scored attention: scores are mixed across at most 64 heads")
    if vd > 512:
        raise KernelError(f"scored attention: value size {vd} is not supported (up to 512)")
    shape = (H, n, vd) if head_major else (n, H, vd)
    if out is None:
        out = torch.empty(shape, dtype=q.dtype, device=q.device)
    elif tuple(out.shape) != shape or out.dtype != q.dtype or out.stride(2) != 1:
        raise KernelError("scored attention: out has the wrong shape, type or strides")
    tok, head = (1, 0) if head_major else (0, 1)
    lib = library("scored_attention")
    if (step is not None and q.dtype == torch.bfloat16 and q.data_ptr() % 16 == 0
            and out.data_ptr() % 4 == 0 and q.stride(tok) % 8 == 0 and q.stride(head) % 8 == 0
            and out.stride(tok) % 2 == 0 and out.stride(head) % 2 == 0
            and lib.gfa_scored_attention_mfma_takes(_i(H), _i(G), _i(hd), _i(vd), _i(int(talk is not None)))):
        q_start, start_pos, n_seqs, max_q_len = step
        require_device(q_start, start_pos)
        require_contiguous(q_start=q_start, start_pos=start_pos)
        if q_start.dtype != torch.int32 or start_pos.dtype != torch.int32 or \
                q_start.numel() < n_seqs + 1 or start_pos.numel() < n_seqs:
            raise KernelError("scored attention: q_start / start_pos must be int32 and cover the batch")
        check(lib.gfa_scored_attention_mfma(
            ptr(q), ptr(k_pages), ptr(v_pages), ptr(q_start), ptr(start_pos), ptr(table),
            _i(table.shape[1]), ptr(temperature), ptr(bias), ptr(lookup if bias is not None else None),
            ptr(talk), ptr(r1), ptr(r2), _i(int(sink)), ptr(out), _i(n_seqs), _i(max_q_len), _i(H),
            _i(G), _i(hd), _i(vd),
            _ll(q.stride(tok)), _ll(q.stride(head)), _ll(out.stride(tok)), _ll(out.stride(head)),
            _f(scale), _f(softcap or 0.0), _i(rows), _i(0 if lookup is None else lookup.numel()),
            _i(window or 0), stream_handle()), "scored_attention_mfma")
        return out
    check(lib.gfa_scored_attention(
        ptr(q), ptr(k_pages), ptr(v_pages), ptr(tok_seq), ptr(tok_pos), ptr(table),
        _i(table.shape[1]), ptr(temperature), ptr(bias), ptr(lookup if bias is not None else None),
        ptr(talk), ptr(r1), ptr(r2), _i(int(sink)), ptr(out), _i(n), _i(H), _i(G), _i(hd), _i(vd),
        _ll(q.stride(tok)),
        _ll(q.stride(head)), _ll(out.stride(tok)), _ll(out.stride(head)), _f(scale),
        _f(softcap or 0.0), _i(rows), _i(0 if lookup is None else lookup.numel()), _i(window or 0),
        _i(_is_bf16(q)), stream_handle()), "scored_attention")
    return out


def unit_heads_store(proj: torch.Tensor, bias: Optional[torch.Tensor], tok_seq, tok_pos, table,
                     k_pages, v_pages, n_heads: int, n_kv_heads: int, head_dim: int, value_dim: int,
                     eps: Optional[float], out_dtype: torch.dtype,
                     q_weight: Optional[torch.Tensor] = None, k_weight: Optional[torch.Tensor] = None,
                     freqs: Optional[torch.Tensor] = None, rotary_dim: int = 0, layout: int = 0,
                     trig_scale: float = 1.0) -> torch.Tensor:
    """q [N, H, d] in ``out_dtype`` from the float32 sums proj [N, >= (H + G) d + G dv] of the
    joined q, k, v projection: the bias added, q and k heads divided by their root mean square
    (``eps`` None: not) and multiplied by ``q_weight`` / ``k_weight`` (float32 [d], shared by the
    heads; None: not), then the first ``rotary_dim`` elements of each head of q and k rotated
    by position times ``freqs`` (float32 [rotary_dim / 2]; layout 0: pairs (2i, 2i + 1), 1:
    pairs (i, i + rotary_dim / 2)) with cos and sin times ``trig_scale``; keys and values put
    into the cache (k_pages None: not)."""
    require_device(proj, bias, tok_seq, tok_pos, table, k_pages, v_pages, q_weight, k_weight, freqs)
    require_contiguous(proj=proj, bias=bias, tok_seq=tok_seq, tok_pos=tok_pos, table=table,
                       q_weight=q_weight, k_weight=k_weight, freqs=freqs)
    width = (n_heads + n_kv_heads) * head_dim + n_kv_heads * value_dim
    if proj.dtype != torch.float32 or proj.dim() != 2 or proj.shape[1] < width:
        raise KernelError(f"unit_heads_store: proj must be float32 [N, >= {width}]")
    if bias is not None and (bias.dtype != torch.float32 or bias.numel() != width):
        raise KernelError(f"unit_heads_store: bias must be float32 [{width}]")
    for name, t in (("q_weight", q_weight), ("k_weight", k_weight)):
        if t is not None and (t.dtype != torch.float32 or t.numel() != head_dim):
            raise KernelError(f"unit_heads_store: {name} must be float32 [{head_dim}]")
    if rotary_dim % 2 or not 0 <= rotary_dim <= head_dim or layout not in (0, 1):
        raise KernelError(f"unit_heads_store: rotary_dim {rotary_dim} must be even and at most {head_dim}")
    if rotary_dim and (freqs is None or freqs.dtype != torch.float32 or freqs.numel() != rotary_dim // 2):
        raise KernelError(f"unit_heads_store: {rotary_dim // 2} float32 frequencies are needed")
    if (k_pages is None) != (v_pages is None):
        raise KernelError("unit_heads_store: give both k_pages and v_pages, or neither")
    _check_pages(k_pages, v_pages, n_kv_heads, head_dim, value_dim, out_dtype)
    n = proj.shape[0]
    if tok_seq.numel() < n or tok_pos.numel() < n:
        raise KernelError("unit_heads_store: token maps are shorter than the batch")
    q = torch.empty((n, n_heads, head_dim), dtype=out_dtype, device=proj.device)
    check(library("scored_attention").gfa_unit_heads_store(
        ptr(proj), _i(proj.shape[1]), ptr(bias), ptr(q), ptr(k_pages), ptr(v_pages), ptr(tok_seq),
        ptr(tok_pos), ptr(table), _i(table.shape[1]), _i(n), _i(n_heads), _i(n_kv_heads),
        _i(head_dim), _i(value_dim), _f(-1.0 if eps is None else eps), ptr(q_weight), ptr(k_weight),
        ptr(freqs if rotary_dim else None), _i(rotary_dim), _i(layout), _f(trig_scale),
        _i(int(out_dtype == torch.bfloat16)), stream_handle()), "unit_heads_store")
    return q


def latent_store(proj: torch.Tensor, q_rank: int, kv_rank: int, rot_dim: int, q_weight, kv_weight,
                 eps: float, freqs: Optional[torch.Tensor], rotary_dim: int, tok_seq, tok_pos, table,
                 k_pages, v_pages, out_dtype: torch.dtype) -> torch.Tensor:
    """The normed query latent [N, q_rank] in ``out_dtype`` from the float32 sums proj
    [N, >= q_rank + kv_rank + rot_dim]; the normed kv latent and the rotated key part go into
    the cache (one kv head; keys of kv_rank + rot_dim, values of kv_rank; None: not)."""
    require_device(proj, q_weight, kv_weight, freqs, tok_seq, tok_pos, table, k_pages, v_pages)
    require_contiguous(proj=proj, q_weight=q_weight, kv_weight=kv_weight, freqs=freqs,
                       tok_seq=tok_seq, tok_pos=tok_pos, table=table)
    width = q_rank + kv_rank + rot_dim
    if proj.dtype != torch.float32 or proj.dim() != 2 or proj.shape[1] < width:
        raise KernelError(f"latent_store: proj must be float32 [N, >= {width}]")
    if (q_rank and (q_weight is None or q_weight.dtype != torch.float32 or q_weight.numel() != q_rank)) \
            or kv_weight.dtype != torch.float32 or kv_weight.numel() != kv_rank:
        raise KernelError("latent_store: the norm weights must be float32 of the latents' sizes")
    if rotary_dim % 2 or rotary_dim > rot_dim:
        raise KernelError(f"latent_store: rotary_dim {rotary_dim} must be even and at most {rot_dim}")
    if rotary_dim and (freqs is None or freqs.dtype != torch.float32 or freqs.numel() != rotary_dim // 2):
        raise KernelError(f"latent_store: {rotary_dim // 2} float32 frequencies are needed")
    if (k_pages is None) != (v_pages is None):
        raise KernelError("latent_store: give both k_pages and v_pages, or neither")
    _check_pages(k_pages, v_pages, 1, kv_rank + rot_dim, kv_rank, out_dtype)
    n = proj.shape[0]
    if tok_seq.numel() < n or tok_pos.numel() < n:
        raise KernelError("latent_store: token maps are shorter than the batch")
    cq = torch.empty((n, q_rank), dtype=out_dtype, device=proj.device)
    check(library("scored_attention").gfa_latent_store(
        ptr(proj), _i(proj.shape[1]), _i(q_rank), _i(kv_rank), _i(rot_dim), ptr(q_weight),
        ptr(kv_weight), _f(eps), ptr(freqs), _i(rotary_dim), ptr(cq), ptr(k_pages), ptr(v_pages),
        ptr(tok_seq), ptr(tok_pos), ptr(table), _i(table.shape[1]), _i(n),
        _i(int(out_dtype == torch.bfloat16)), stream_handle()), "latent_store")
    return cq


def whole_norm_store(proj: torch.Tensor, bias: Optional[torch.Tensor], q_weight, k_weight, tok_seq,
                     tok_pos, table, k_pages, v_pages, n_heads: int, n_kv_heads: int, head_dim: int,
                     value_dim: int, eps: Optional[float], temp_coef: Optional[float],
                     temp_every: int, values_are_keys: bool, out_dtype: torch.dtype) -> torch.Tensor:
    """q [N, H, d] in ``out_dtype`` from the float32 sums proj [N, >= (H + G) d (+ G dv)] of the
    joined projection: the bias added; all of q, and all of k, divided by the root mean square
    of the whole projection and multiplied by a weight per element (``eps`` None: not); q times
    ``1 + temp_coef ln(floor((pos + 1) / temp_every) + 1)`` (``temp_coef`` None: not); the
    normed keys go into the cache, and as values either the keys as projected
    (``values_are_keys``) or the row's third part (k_pages None: nothing is stored)."""
    require_device(proj, bias, q_weight, k_weight, tok_seq, tok_pos, table, k_pages, v_pages)
    require_contiguous(bias=bias, q_weight=q_weight, k_weight=k_weight, tok_seq=tok_seq,
                       tok_pos=tok_pos, table=table)
    nq, nk = n_heads * head_dim, n_kv_heads * head_dim
    width = nq + nk + (0 if values_are_keys else n_kv_heads * value_dim)
    if proj.dtype != torch.float32 or proj.dim() != 2 or proj.shape[1] < width or proj.stride(1) != 1:
        raise KernelError(f"whole_norm_store: proj must be float32 [N, >= {width}]")
    if bias is not None and (bias.dtype != torch.float32 or bias.numel() != width):
        raise KernelError(f"whole_norm_store: bias must be float32 [{width}]")
    if values_are_keys and value_dim != head_dim:
        raise KernelError("whole_norm_store: values that are the keys have the keys' size")
    if eps is not None:
        for name, t, count in (("q_weight", q_weight, nq), ("k_weight", k_weight, nk)):
            if t is None or t.dtype != torch.float32 or t.numel() != count:
                raise KernelError(f"whole_norm_store: {name} must be float32 [{count}]")
    if temp_coef is not None and temp_every < 1:
        raise KernelError("whole_norm_store: temp_every must be at least 1")
    if (k_pages is None) != (v_pages is None):
        raise KernelError("whole_norm_store: give both k_pages and v_pages, or neither")
    _check_pages(k_pages, v_pages, n_kv_heads, head_dim, value_dim, out_dtype)
    n = proj.shape[0]
    if tok_seq.numel() < n or tok_pos.numel() < n:
        raise KernelError("whole_norm_store: token maps are shorter than the batch")
    q = torch.empty((n, n_heads, head_dim), dtype=out_dtype, device=proj.device)
    check(library("scored_attention").gfa_whole_norm_store(
        ptr(proj), _i(proj.stride(0)), ptr(bias), ptr(q_weight), ptr(k_weight), ptr(q), ptr(k_pages),
        ptr(v_pages), ptr(tok_seq), ptr(tok_pos), ptr(table), _i(table.shape[1]), _i(n), _i(n_heads),
        _i(n_kv_heads), _i(head_dim), _i(value_dim), _f(-1.0 if eps is None else eps),
        _f(0.0 if temp_coef is None else temp_coef), _i(0 if temp_coef is None else temp_every),
        _i(int(values_are_keys)), _i(int(out_dtype == torch.bfloat16)), stream_handle()),
        "whole_norm_store")
    return q


def latent_query(q: torch.Tensor, freqs: Optional[torch.Tensor], rotary_dim: int, tok_pos,
                 n_heads: int, head_dim: int, rot_dim: int, kv_rank: int, out_dtype: torch.dtype):
    """From the float32 sums q [N, H (d + dr)] of the query's up projection: the plain parts
    head by head, [H, N, d], and a tensor [H, N, kv_rank + dr] whose last dr elements hold the
    rotated parts (the first kv_rank are left for the product with the keys' up projection)."""
    require_device(q, freqs, tok_pos)
    require_contiguous(freqs=freqs, tok_pos=tok_pos)
    n = q.shape[0]
    if q.dtype != torch.float32 or q.dim() != 2 or q.shape[1] != n_heads * (head_dim + rot_dim) \
            or q.stride(1) != 1:
        raise KernelError(f"latent_query: q must be float32 [N, {n_heads * (head_dim + rot_dim)}] "
                          f"with unit stride along a row (a view of wider rows is allowed)")
    if rotary_dim % 2 or rotary_dim > rot_dim:
        raise KernelError(f"latent_query: rotary_dim {rotary_dim} must be even and at most {rot_dim}")
    if rotary_dim and (freqs is None or freqs.dtype != torch.float32 or freqs.numel() != rotary_dim // 2):
        raise KernelError(f"latent_query: {rotary_dim // 2} float32 frequencies are needed")
    if tok_pos.numel() < n or tok_pos.dtype != torch.int32:
        raise KernelError("latent_query: tok_pos must be int32 and cover the batch")
    plain = torch.empty((n_heads, n, head_dim), dtype=out_dtype, device=q.device)
    full = torch.empty((n_heads, n, kv_rank + rot_dim), dtype=out_dtype, device=q.device)
    check(library("scored_attention").gfa_latent_query(
        ptr(q), ptr(freqs), _i(rotary_dim), ptr(tok_pos), ptr(plain), ptr(full), _i(n), _i(n_heads),
        _i(head_dim), _i(rot_dim), _i(kv_rank), _ll(q.stride(0)),
        _i(int(out_dtype == torch.bfloat16)), stream_handle()), "latent_query")
    return plain, full
