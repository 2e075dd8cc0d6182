"""Refolix on the GPU against the plain float64 implementation of tests/plain_refolix.py: each
mechanism's kernels alone (the layer norm and the join that norms after the sum, heads that
are normed, rotated and stored, attention with a window and a cap, the short convolutions with
their tails, the delta rule with carried state, the rotation of rows, the norm per head with
its gate, the router with its correction and the gated experts in each of their forms), whole
prompts with the stream after every layer, prompts in portions, token-by-token decoding,
unequal batches, slots and pages that come back, keys at a window's edge and at page borders
with inputs that make one key stand out, state that lasts for hundreds of tokens, long
decoding, and greedy generation through the library's generation loop, command line and trace
replay."""
import math
import os

import pytest
import torch

import plain_refolix as P
import util
from refolix_cases import CASES, make_folder, random_case, write_model
from util import TOL_BF16, rel_err

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
F = torch.float64
# float32 engine against float64 over a few hundred tokens and several norms
TOL_F32_LONG = 1e-4


def row_errors(got, want):
    """Per row: root mean square of the difference over that of all of ``want``."""
    got, want = got.double().cpu(), want.double().cpu()
    return (got - want).pow(2).mean(-1).sqrt() / want.pow(2).mean().sqrt()


def bf16_close(got, want):
    """A bfloat16 engine against float64: every sum is normed, a head's result is divided by
    its own root mean square, and a router's close call may fall the other way after a
    rounding, so single rows can be off by more than the typical one.  The typical row is held
    to the tolerance and all but one in a hundred (at least one) to a bound that a wrong key, a
    lost state or a missing term, which touch most rows, would break.  The float32 engine is
    the sharp test."""
    e = row_errors(got, want).sort().values
    rest = e[:max(1, e.numel() - max(1, e.numel() // 100))]
    return float(rest.max()) < 0.3 and float(e.median()) < TOL_BF16


def close(got, want, dtype, tol):
    return bf16_close(got, want) if dtype == "bfloat16" else rel_err(got, want) < tol


def _engine(folder, dtype, **kw):
    import gpt_fast_amd as gfa
    kw.setdefault("max_tokens", 4096)
    return gfa.Engine.from_folder(folder, dtype=dtype, device=DEV, **kw)


def _steps(eng, toks, cuts):
    """Feed ``toks`` as one sequence in portions that end at ``cuts``; logits of every token."""
    import gpt_fast_amd as gfa
    slot = eng.start_sequence()
    out, lo = [], 0
    for hi in list(cuts) + [len(toks)]:
        if hi <= lo:
            continue
        out.append(eng.step([gfa.Entry(slot, toks[lo:hi], want=list(range(hi - lo)))]).cpu())
        lo = hi
    eng.end_sequence(slot)
    return torch.cat(out)


def _ints(values):
    return torch.tensor(values, dtype=torch.int32, device=DEV)


def _f32(t):
    return t.to(torch.float32).to(DEV).contiguous()


def _table_and_positions(lens, starts):
    """Pages handed out in reverse; the step's token maps."""
    total = [s + l for s, l in zip(starts, lens)]
    n_pages = sum((t + 63) // 64 for t in total)
    order, tables, at = list(range(n_pages))[::-1], [], 0
    for t in total:
        n = (t + 63) // 64
        tables.append(order[at:at + n])
        at += n
    widest = max(len(t) for t in tables)
    table = _ints([t + [-1] * (widest - len(t)) for t in tables])
    tok_seq = _ints([b for b, l in enumerate(lens) for _ in range(l)])
    pos = [s + i for s, l in zip(starts, lens) for i in range(l)]
    return n_pages, tables, table, tok_seq, _ints(pos), pos


def _cache_rows(k_pages, v_pages, d, dv):
    """What the kernels keep -> keys [n, G, 64, d] and values [n, G, dv, 64]."""
    n, G = k_pages.shape[:2]
    k = k_pages.reshape(n, G, -1)[..., util.key_places(d).reshape(-1)].view(n, G, 64, d)
    v = v_pages.reshape(n, G, -1)[..., util.value_places(dv).reshape(-1)].view(n, G, dv, 64)
    return k.double().cpu(), v.double().cpu()


# --------------------------------------------------------------------------- norms and joins
@pytest.mark.parametrize("dim", [50, 96, 1030, 4096, 8200])
def test_the_layer_norm_and_the_join_that_norms_after_the_sum(dim):
    from gpt_fast_amd.ops import kernels as K
    g = torch.Generator().manual_seed(dim)
    n = 7
    x = torch.randn(n, dim, generator=g, dtype=F) * 3 + 0.7            # a mean that matters
    y, y2 = torch.randn(n, dim, generator=g, dtype=F), torch.randn(n, dim, generator=g, dtype=F) * 5
    w, ls, wa, wb = (torch.rand(dim, generator=g, dtype=F) + 0.5 for _ in range(4))
    eps = 1e-5
    rows = _ints([5, 0, 5, 3])
    got = K.layer_norm(_f32(x), _f32(w), eps, torch.float32, rows=rows)
    assert rel_err(got, P.layer_norm(x[[5, 0, 5, 3]], w, eps)) < 1e-5
    got = K.layer_norm(_f32(x), _f32(w), eps, torch.bfloat16)
    assert rel_err(got, P.layer_norm(x, w, eps)) < 1e-2
    # one result
    res = _f32(x)
    out = K.post_norm_join(res, _f32(y), _f32(w), eps, alpha=2.5, layer_scale=_f32(ls), out_dtype=torch.bfloat16)
    want = P.layer_norm(2.5 * x + ls * y, w, eps)
    assert rel_err(res, want) < 1e-5 and rel_err(out, want) < 1e-2
    # no layer scale, no rows for a reader
    res = _f32(x)
    assert K.post_norm_join(res, _f32(y), _f32(w), eps) is None
    assert rel_err(res, P.layer_norm(x + y, w, eps)) < 1e-5
    # two branches, each over its root mean square, averaged
    res = _f32(x)
    out = K.post_norm_join(res, _f32(y), _f32(w), eps, alpha=0.5, layer_scale=_f32(ls), second=_f32(y2),
                           branch_weights=(_f32(wa), _f32(wb)), branch_eps=1e-3, out_dtype=torch.float32)
    mixed = 0.5 * (P.unit_rms(y, 1e-3) * wa + P.unit_rms(y2, 1e-3) * wb)
    want = P.layer_norm(0.5 * x + ls * mixed, w, eps)
    assert rel_err(res, want) < 1e-5 and rel_err(out, want) < 1e-5


# --------------------------------------------------------------------------- heads normed, rotated, stored
@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-5), (torch.bfloat16, 1e-2)])
@pytest.mark.parametrize("H,G,d,dv,dims,layout,scaling", [
    (4, 2, 16, 16, 8, "interleaved", (4.0, 64, 16.0, 2.0)), (3, 3, 20, 12, 20, "half", None),
    (6, 1, 8, 32, 2, "interleaved", None), (2, 1, 10, 6, 6, "half", (3.0, 40, 8.0, 1.0)),
    (2, 2, 24, 8, 0, "interleaved", None)])
def test_heads_are_normed_weighted_rotated_and_stored(dtype, tol, H, G, d, dv, dims, layout, scaling):
    from gpt_fast_amd.config.spec import PositionSpec
    from gpt_fast_amd.ops import scored_attention as SA
    from gpt_fast_amd.parts.position import RotaryPosition, frequencies_and_trig_scale
    g = torch.Generator().manual_seed(H * 100 + d)
    lens, starts = [5, 1, 70], [0, 63, 130]
    n_pages, tables, table, tok_seq, tok_pos, pos = _table_and_positions(lens, starts)
    N = sum(lens)
    width = (H + G) * d + G * dv
    proj = torch.randn(N, width + 3, generator=g, dtype=F)
    wq, wk = torch.rand(d, generator=g, dtype=F) + 0.5, torch.rand(d, generator=g, dtype=F) + 0.5
    rot = {"dims": dims, "base": 100.0}
    freqs, trig, lay = None, 1.0, 0
    if dims:
        sc = None
        if scaling is not None:
            rot["scaling"] = dict(zip(("factor", "original", "fast", "slow"), scaling))
            sc = (("rope_type", "yarn"),) + tuple(rot["scaling"].items())
        freqs, trig = frequencies_and_trig_scale(PositionSpec(rotary_dim=dims, base=100.0, layout=layout, scaling=sc))
        assert rel_err(freqs, P.rotary_frequencies(rot)[0]) < 1e-6 and abs(trig - P.rotary_frequencies(rot)[1]) < 1e-12
        freqs, lay = freqs.to(DEV), RotaryPosition.LAYOUTS[layout]
    k_pages = torch.zeros(n_pages, G, 64, d, dtype=dtype, device=DEV)
    v_pages = torch.zeros(n_pages, G, dv, 64, dtype=dtype, device=DEV)
    q = SA.unit_heads_store(_f32(proj), None, tok_seq, tok_pos, table, k_pages, v_pages, H, G, d, dv, 1e-5,
                            dtype, q_weight=_f32(wq), k_weight=_f32(wk), freqs=freqs, rotary_dim=dims,
                            layout=lay, trig_scale=trig)
    p = torch.tensor(pos)
    wq_ = P.rotate(P.unit_rms(proj[:, :H * d].view(N, H, d), 1e-5) * wq, p, rot, layout)
    wk_ = P.rotate(P.unit_rms(proj[:, H * d:(H + G) * d].view(N, G, d), 1e-5) * wk, p, rot, layout)
    wv_ = proj[:, (H + G) * d:width].view(N, G, dv)
    assert rel_err(q, wq_) < tol
    keys, values = _cache_rows(k_pages, v_pages, d, dv)
    for n in range(N):
        b = int(tok_seq[n])
        page = tables[b][pos[n] // 64]
        assert rel_err(keys[page, :, pos[n] % 64], wk_[n]) < tol
        assert rel_err(values[page, :, :, pos[n] % 64], wv_[n]) < tol


# --------------------------------------------------------------------------- attention with a window
def _plain_window_attention(q, k, v, start, scale, cap, window):
    """q [L, H, d] at positions start..; k [T, G, d], v [T, G, dv] of the whole sequence."""
    L, H, _ = q.shape
    G = k.shape[1]
    out = torch.zeros(L, H, v.shape[2], dtype=F)
    for i in range(L):
        pos = start + i
        lo = 0 if not window else max(0, pos - window + 1)
        for h in range(H):
            s = (k[lo:pos + 1, h // (H // G)] @ q[i, h]) * scale
            if cap:
                s = cap * torch.tanh(s / cap)
            out[i, h] = torch.softmax(s, 0) @ v[lo:pos + 1, h // (H // G)]
    return out


def _attention_alone(dtype, H, G, d, dv, lens, starts, window, cap, scale=0.3, loud=None, seed=0):
    """Keys and values of whole sequences put into pages (handed out in reverse) by the storing
    kernel, then the step's tokens attend.  ``loud`` = (sequence, key position): that key is
    made so that it takes all the weight of that sequence's queries wherever it is seen."""
    from gpt_fast_amd.ops import scored_attention as SA
    g = torch.Generator().manual_seed(seed + H + d)
    total = [s + l for s, l in zip(starts, lens)]
    n_pages, tables, table, _, _, _ = _table_and_positions(total, [0] * len(total))
    ks = [torch.randn(t, G, d, generator=g, dtype=F) for t in total]
    vs = [torch.randn(t, G, dv, generator=g, dtype=F) for t in total]
    qs = [torch.randn(l, H, d, generator=g, dtype=F) for l in lens]
    if loud is not None:
        # every query of that sequence looks for the key's first element, which that key alone has
        b, j = loud
        qs[b][:, :, 0] = 3.0
        ks[b][:, :, 0] = 0.0
        ks[b][j, :, 0] = 30.0
    if dtype == torch.bfloat16:
        ks, vs, qs = ([t.to(dtype).double() for t in ts] for ts in (ks, vs, qs))
    k_pages = torch.full((n_pages + 1, G, 64, d), float("nan"), dtype=dtype, device=DEV)
    v_pages = torch.full((n_pages + 1, G, dv, 64), float("nan"), dtype=dtype, device=DEV)
    rows = torch.cat([torch.cat([torch.zeros(t, H * d, dtype=F), k.reshape(t, -1), v.reshape(t, -1)], 1)
                      for t, k, v in zip(total, ks, vs)])
    seq_all = _ints([b for b, t in enumerate(total) for _ in range(t)])
    pos_all = _ints([i for t in total for i in range(t)])
    SA.unit_heads_store(_f32(rows), None, seq_all, pos_all, table, k_pages, v_pages, H, G, d, dv, None, dtype)
    tok_seq = _ints([b for b, l in enumerate(lens) for _ in range(l)])
    tok_pos = _ints([s + i for s, l in zip(starts, lens) for i in range(l)])
    q_start = _ints([sum(lens[:b]) for b in range(len(lens) + 1)])
    q = torch.cat(qs).to(dtype).to(DEV)
    results = []
    for step in (None, (q_start, _ints(starts), len(lens), max(lens))):
        got = SA.attention(q, k_pages, v_pages, tok_seq, tok_pos, table, scale, window=window or 0,
                           softcap=cap or 0.0, step=step)
        results.append(got.double().cpu())
    want = torch.cat([_plain_window_attention(qq, k, v, s, scale, cap, window)
                      for qq, k, v, s in zip(qs, ks, vs, starts)])
    return results, want, vs


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-5), (torch.bfloat16, 2e-2)])
@pytest.mark.parametrize("H,G,d,dv,window,cap", [(4, 2, 16, 32, 40, 5.0), (3, 3, 24, 16, 64, None), (8, 1, 8, 16, 1, 2.0),
                                                 (2, 1, 10, 6, 33, 9.0), (4, 4, 32, 48, None, 30.0), (6, 2, 96, 48, 100, 20.0)])
def test_attention_with_a_window_and_a_cap_alone(dtype, tol, H, G, d, dv, window, cap):
    # a prompt, a portion at an offset that a window's start falls into, single tokens
    for lens, starts in (([150, 3], [0, 0]), ([37, 2, 1], [100, 63, 64]), ([1, 1, 1, 1], [0, 63, 64, 200])):
        results, want, _ = _attention_alone(dtype, H, G, d, dv, lens, starts, window, cap)
        for got in results:
            assert rel_err(got, want) < tol, (lens, starts)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("window", [1, 2, 40, 64, 65, 130])
def test_a_key_just_inside_and_just_outside_the_window_in_prompts_and_single_tokens(dtype, window):
    """One key is made so loud that it takes all the weight wherever it is seen: the query at
    distance window - 1 returns that key's value, the one at distance window does not."""
    H, G, d, dv = 4, 2, 16, 16
    for key in (0, 5, 63, 64, 127, 128):
        inside, outside = key + window - 1, key + window
        for lens, starts in (([outside + 3], [0]), ([4], [inside - 1]), ([1, 1], [inside, outside])):
            total = max(s + l for s, l in zip(starts, lens))
            if total <= outside or min(starts) < 0:
                continue
            results, want, vs = _attention_alone(dtype, H, G, d, dv, lens, starts, window, None, scale=1.0,
                                                 loud=(0, key), seed=key)
            for got in results:
                assert rel_err(got, want) < (2e-5 if dtype == torch.float32 else 3e-2)
            # the plain result itself shows the edge: the loud key's value inside, not outside
            if len(lens) == 1 and starts[0] == 0 and window > 1:
                assert rel_err(want[inside, 0], vs[0][key, 0]) < 1e-3
                assert rel_err(want[outside, 0], vs[0][key, 0]) > 0.1


# --------------------------------------------------------------------------- convolutions and the delta rule
def _delta_reference(x_q, x_k, x_v, taps, b_pre, a_pre, A_log, dt_bias, H, G, dk, dv):
    """Whole sequences: convolution, silu, unit vectors, the recurrence; o [T, H, dv]."""
    T = x_q.shape[0]
    C1 = G * dk
    q = P.silu(P.short_convolution(x_q, taps[:C1])).view(T, G, dk)
    k = P.silu(P.short_convolution(x_k, taps[C1:2 * C1])).view(T, G, dk)
    v = P.silu(P.short_convolution(x_v, taps[2 * C1:])).view(T, H, dv)
    conv = torch.cat([q.reshape(T, -1), k.reshape(T, -1), v.reshape(T, -1)], 1)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * dk ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(b_pre)
    gate = torch.exp(-torch.exp(A_log) * P.softplus(a_pre + dt_bias))
    o = torch.zeros(T, H, dv, dtype=F)
    for h in range(H):
        S = torch.zeros(dk, dv, dtype=F)
        for t in range(T):
            S = gate[t, h] * S
            u = beta[t, h] * (v[t, h] - S.T @ k[t, h // (H // G)])
            S = S + torch.outer(k[t, h // (H // G)], u)
            o[t, h] = S.T @ q[t, h // (H // G)]
    return conv, o


@pytest.mark.parametrize("chunked", [0, 32, 64])
@pytest.mark.parametrize("H,G,dk,dv,K_", [(4, 2, 16, 8, 3), (1, 1, 32, 40, 5), (3, 3, 12, 20, 1), (6, 2, 8, 64, 2),
                                          (2, 1, 128, 96, 4), (2, 2, 70, 33, 4)])
def test_the_convolutions_tails_and_the_delta_rule_with_carried_state(H, G, dk, dv, K_, chunked):
    """Three sequences in scattered slots, fed in portions of unequal sizes (down to one and two
    tokens, shorter than the taps); state and tails travel from step to step; token by token,
    and a chunk of 32 or of 64 tokens at a time."""
    from gpt_fast_amd.ops import gated_delta as GD
    g = torch.Generator().manual_seed(H * 31 + dk)
    layout = GD.RowLayout.fused(H, G, dk, dv)
    C = layout.conv
    lens = [75, 9, 40]
    slots = [5, 0, 3]
    proj = [torch.randn(n, layout.width, generator=g, dtype=F) for n in lens]
    taps = torch.randn(C, K_, generator=g, dtype=F) * 0.7
    A_log, dt_bias = torch.rand(H, generator=g, dtype=F) * 4 - 4, torch.randn(H, generator=g, dtype=F)
    size = GD.state_size(H, G, dk, dv, K_)
    state = torch.zeros(7, size, dtype=torch.float32, device=DEV)
    state[1].fill_(float("nan"))                                     # a slot nobody owns
    tail_off = H * dk * dv
    plans = [[1, 2, 30, 2, 40], [2, 1, 1, 5], [40]]                  # portions per sequence
    fed = [0, 0, 0]
    conv_got = [[] for _ in lens]
    o_got = [[] for _ in lens]
    step = 0
    while any(fed[b] < lens[b] for b in range(3)):
        live = [b for b in range(3) if fed[b] < lens[b] and step < len(plans[b])]
        take = [plans[b][step] for b in live]
        rows = torch.cat([proj[b][fed[b]:fed[b] + n] for b, n in zip(live, take)])
        q_start = _ints([sum(take[:i]) for i in range(len(take) + 1)])
        tok_seq = _ints([i for i, n in enumerate(take) for _ in range(n)])
        sl = _ints([slots[b] for b in live])
        rows_dev = _f32(rows)
        conv = GD.short_conv(rows_dev, layout, _f32(taps), state, tail_off, tok_seq, q_start, sl, len(live))
        o = GD.scan(conv, rows_dev, layout, _f32(A_log), _f32(dt_bias), state, q_start, sl, len(live),
                    H, G, dk, dv, dk ** -0.5, 1e-6, chunked=bool(chunked), max_q_len=chunked)
        at = 0
        for b, n in zip(live, take):
            conv_got[b].append(conv[at:at + n].double().cpu())
            o_got[b].append(o[at:at + n].double().cpu())
            at += n
            fed[b] += n
        step += 1
    C1 = G * dk
    for b in range(3):
        x = proj[b]
        conv, o = _delta_reference(x[:, :C1], x[:, C1:2 * C1], x[:, 2 * C1:C], taps, x[:, layout.b:layout.b + H],
                                   x[:, layout.a:layout.a + H], A_log, dt_bias, H, G, dk, dv)
        assert rel_err(torch.cat(conv_got[b]), conv) < 1e-5, b
        assert rel_err(torch.cat(o_got[b]).view(-1, H, dv), o) < 2e-4, b
        # the tail holds the sequence's last inputs, oldest first
        if K_ > 1:
            tail = state[slots[b], tail_off:tail_off + (K_ - 1) * C].view(K_ - 1, C).double().cpu()
            assert rel_err(tail, x[-(K_ - 1):, :C]) < 1e-6
    assert torch.isnan(state[1]).all()


def test_the_delta_rule_forgets_and_overwrites_as_its_equations_say():
    """beta = 1 and no decay: writing value v under key k and asking with q = k returns v; a
    second write under the same key replaces the first; with decay 0 nothing earlier is left."""
    from gpt_fast_amd.ops import gated_delta as GD
    H = G = 1
    dk, dv = 8, 4
    layout = GD.RowLayout.fused(H, G, dk, dv)
    T = 3
    conv = torch.zeros(T, layout.conv, dtype=F)
    key = torch.zeros(dk, dtype=F)
    key[2] = 3.0
    other = torch.zeros(dk, dtype=F)
    other[5] = 1.0
    values = torch.tensor([[1.0, 2.0, 3.0, 4.0], [9.0, 8.0, 7.0, 6.0], [0.5, 0.5, 0.5, 0.5]], dtype=F)
    for t, (qq, kk) in enumerate([(key, key), (key, key), (key, other)]):
        conv[t, :dk], conv[t, dk:2 * dk], conv[t, 2 * dk:] = qq, kk, values[t]
    proj = torch.zeros(T, layout.width, dtype=F)
    proj[:, layout.b] = 40.0                           # beta = 1
    proj[:, layout.a] = -40.0                          # softplus = 0: no decay
    state = torch.zeros(2, GD.state_size(H, G, dk, dv, 1), dtype=torch.float32, device=DEV)
    o = GD.scan(_f32(conv), _f32(proj), layout, _f32(torch.zeros(1)), _f32(torch.zeros(1)), state,
                _ints([0, T]), _ints([0]), 1, H, G, dk, dv, 1.0, 0.0).double().cpu()
    assert rel_err(o[0], values[0]) < 1e-5             # read back what was just written
    assert rel_err(o[1], values[1]) < 1e-5             # the same key: replaced, not added
    assert rel_err(o[2], values[1]) < 1e-5             # another key leaves it alone
    proj[:, layout.a] = 40.0                           # a decay of exp(-40): everything is forgotten
    state.zero_()
    conv[2, dk:2 * dk] = other
    o = GD.scan(_f32(conv), _f32(proj), layout, _f32(torch.zeros(1)), _f32(torch.zeros(1)), state,
                _ints([0, T]), _ints([0]), 1, H, G, dk, dv, 1.0, 0.0).double().cpu()
    assert float(o[2].abs().max()) < 1e-6


@pytest.mark.parametrize("layout", ["interleaved", "half"])
def test_rows_are_rotated_in_place_and_multiplied(layout):
    from gpt_fast_amd.ops import kernels as K
    g = torch.Generator().manual_seed(4)
    N, H, hd, dims, off = 9, 3, 20, 12, 7
    x = torch.randn(N, off + H * hd + 5, generator=g, dtype=F)
    pos = [0, 1, 2, 63, 64, 65, 500, 1000, 4000]
    rot = {"dims": dims, "base": 1000.0}
    f, _ = P.rotary_frequencies(rot)
    dev = _f32(x)
    K.rotate_rows(dev, off, H, hd, dims, 0 if layout == "interleaved" else 1, _f32(f), _ints(pos), 1.0, 0.25)
    want = x.clone()
    want[:, off:off + H * hd] = (P.rotate(x[:, off:off + H * hd].reshape(N, H, hd), torch.tensor(pos), rot, layout)
                                 * 0.25).reshape(N, -1)
    assert rel_err(dev, want) < 1e-4          # float32 angles of some thousand radians
    # the heads from the third on with a factor of their own, in the same call
    dev = _f32(x)
    K.rotate_rows(dev, off, H, hd, dims, 0 if layout == "interleaved" else 1, _f32(f), _ints(pos), 1.0, 1.0,
                  late_from=2, late_factor=0.5)
    turned = P.rotate(x[:, off:off + H * hd].reshape(N, H, hd), torch.tensor(pos), rot, layout)
    turned[:, 2:] *= 0.5
    want[:, off:off + H * hd] = turned.reshape(N, -1)
    assert rel_err(dev, want) < 1e-4


@pytest.mark.parametrize("groups,weight,gate", [(1, "row", "sigmoid"), (4, "head", "silu"), (4, None, "silu"),
                                                (2, "row", "silu")])
def test_the_norm_over_rows_or_heads_with_its_gate(groups, weight, gate):
    from gpt_fast_amd.ops import decayed_memory as M
    g = torch.Generator().manual_seed(groups)
    N, W = 6, 48
    o = torch.randn(N, W, generator=g, dtype=F) * 2
    proj = torch.randn(N, 2 * W, generator=g, dtype=F)
    w = None if weight is None else torch.rand(W if weight == "row" else W // groups, generator=g, dtype=F) + 0.5
    layout = M.RowLayout(2 * W, 0, 0, 0, W)
    got = M.row_norm_gate(_f32(o), None if w is None else _f32(w), _f32(proj), layout, 1e-5, torch.float32,
                          groups=groups, gate=gate)
    normed = P.unit_rms(o.view(N, groups, -1), 1e-5)
    if w is not None:
        normed = normed * (w if weight == "head" else w.view(groups, -1))
    gv = proj[:, W:]
    want = normed.reshape(N, W) * (torch.sigmoid(gv) if gate == "sigmoid" else P.silu(gv))
    assert rel_err(got, want) < 1e-5


# --------------------------------------------------------------------------- retention alone
@pytest.mark.parametrize("H,dk,dv,dims", [(3, 16, 24, 16), (2, 24, 8, 12), (1, 20, 12, 0), (2, 8, 144, 8)])
def test_retention_with_carried_state_chunked_and_token_by_token(H, dk, dv, dims):
    """The mixer's cell as the part runs it: rotation of the projection's rows, the key's
    factor, then the decayed state, over portions of many tokens and of one."""
    from gpt_fast_amd.ops import decayed_memory as M
    from gpt_fast_amd.ops import kernels as K
    g = torch.Generator().manual_seed(H + dk)
    T = 200
    layout = M.RowLayout.fused(H, dk, dv)
    proj = torch.randn(T, layout.width, generator=g, dtype=F)
    decay = [1.0 - 2.0 ** -(2 + 2 * h) for h in range(H)]
    rot = {"dims": dims, "base": 500.0}
    pos = torch.arange(T)
    q = P.rotate(proj[:, :H * dk].reshape(T, H, dk), pos, rot, "half")
    k = P.rotate(proj[:, H * dk:2 * H * dk].reshape(T, H, dk), pos, rot, "half") * dk ** -0.5
    v = proj[:, layout.v:layout.v + H * dv].reshape(T, H, dv)
    want = torch.zeros(T, H, dv, dtype=F)
    for h in range(H):
        S = torch.zeros(dk, dv, dtype=F)
        for t in range(T):
            S = decay[h] * S + torch.outer(k[t, h], v[t, h])
            want[t, h] = S.T @ q[t, h]
    freqs = _f32(P.rotary_frequencies(rot)[0]) if dims else None
    state = torch.zeros(3, M.state_size(H, dk, dv), dtype=torch.float32, device=DEV)
    got, lo = [], 0
    for hi in (70, 71, 73, 140, 200):
        rows = _f32(proj[lo:hi])
        tok_pos = _ints(list(range(lo, hi)))
        K.rotate_rows(rows, layout.q, H, dk, dims, 1, freqs, tok_pos, 1.0, 1.0)
        K.rotate_rows(rows, layout.k, H, dk, dims, 1, freqs, tok_pos, 1.0, dk ** -0.5)
        got.append(M.cell(rows, layout, _f32(torch.tensor(decay)), state, _ints([0, hi - lo]), _ints([2]), 1,
                          hi - lo, H, dk, dv, activation=False).double().cpu())
        lo = hi
    assert rel_err(torch.cat(got).view(T, H, dv), want) < 2e-4


# --------------------------------------------------------------------------- the router and the experts
@pytest.mark.parametrize("E,top,groups,keep", [(6, 2, 3, 2), (4, 1, 2, 1), (8, 3, 4, 2), (5, 2, 1, 1), (3, 3, 1, 1),
                                               (6, 2, 6, 3), (16, 4, 4, 1), (12, 4, 2, 2)])
def test_the_router_scores_by_sigmoid_corrects_the_choice_and_keeps_groups(E, top, groups, keep):
    from gpt_fast_amd.ops import routed_experts as RE
    g = torch.Generator().manual_seed(E * 10 + top)
    z = torch.randn(50, E + 3, generator=g, dtype=F) * 2
    corr = torch.randn(E, generator=g, dtype=F) * 0.6 - 0.6        # most choice scores are negative
    chosen, weights = RE.route(_f32(z)[:, :E], E, top, groups, keep, 1e-20, scoring="sigmoid",
                               correction=_f32(corr), group_top=2)
    want_c, want_w = P.route(z[:, :E].float().double(), corr.float().double(), top, groups, keep)
    assert (chosen.cpu().sort(-1).values == want_c.sort(-1).values).all()
    order = chosen.cpu().long().argsort(-1), want_c.argsort(-1)
    assert rel_err(weights.cpu().gather(1, order[0]), want_w.gather(1, order[1])) < 1e-5


def test_the_router_by_hand():
    """Six experts in three groups of two, two groups kept, top 2.  Scores s = sigmoid(z); the
    correction lifts expert 4 over expert 0 in the choice but not in the weights; the group of
    the single best expert loses against two groups with two fair experts each."""
    from gpt_fast_amd.ops import routed_experts as RE
    s = torch.tensor([[0.60, 0.50, 0.90, 0.05, 0.55, 0.45]], dtype=F)
    z = torch.log(s / (1 - s))
    corr = torch.tensor([0.0, 0.0, 0.0, 0.0, 0.1, 0.0], dtype=F)
    # group scores: 1.10, 0.95, 1.10 (with the correction) -> groups 0 and 2; of their experts the
    # choice scores are 0.60, 0.50, 0.65, 0.45 -> experts 4 and 0; weights from s: 0.55, 0.60
    chosen, weights = RE.route(_f32(z), 6, 2, 3, 2, 1e-20, scoring="sigmoid", correction=_f32(corr), group_top=2)
    assert chosen.cpu().tolist() == [[4, 0]]
    assert rel_err(weights, torch.tensor([[0.55 / 1.15, 0.60 / 1.15]])) < 1e-5
    # with the largest score as a group's score, group 1 (0.90) is kept and expert 2 chosen first
    chosen, _ = RE.route(_f32(z), 6, 2, 3, 2, 1e-20, scoring="sigmoid", correction=_f32(corr), group_top=1)
    assert chosen.cpu().tolist() == [[2, 4]]
    # negative choice scores: an expert outside the kept groups is never better than one inside
    corr = torch.tensor([-5.0, -5.0, 0.0, 0.0, -5.0, -5.0], dtype=F)
    chosen, _ = RE.route(_f32(z), 6, 2, 3, 1, 1e-20, scoring="sigmoid", correction=_f32(corr), group_top=2)
    assert sorted(chosen.cpu().tolist()[0]) == [2, 3]
    corr = torch.tensor([-5.0, -5.0, -9.0, -9.0, -9.0, -9.0], dtype=F)
    chosen, _ = RE.route(_f32(z), 6, 2, 3, 1, 1e-20, scoring="sigmoid", correction=_f32(corr), group_top=2)
    assert sorted(chosen.cpu().tolist()[0]) == [0, 1]


@pytest.mark.parametrize("dtype,tol", [("float32", 1e-5), ("bfloat16", 2e-2)])
@pytest.mark.parametrize("D,E,top,groups,keep,F_,shared", [(72, 6, 2, 3, 2, 40, 56), (104, 4, 1, 2, 1, 24, 0),
                                                           (100, 4, 2, 2, 1, 18, 10), (64, 6, 2, 6, 3, 24, 16)])
def test_the_mixture_of_gated_experts_alone_at_every_number_of_rows(dtype, tol, D, E, top, groups, keep, F_, shared):
    """The feed-forward part by itself, with 1 to 150 rows (every form of the experts'
    products), in a step of single tokens and in a prompt, against every expert run densely."""
    import types
    from gpt_fast_amd.config.spec import RoutedExpertsSpec
    from gpt_fast_amd.parts.base import FEED_FORWARDS, Runtime
    g = torch.Generator().manual_seed(D + E)
    dt = torch.bfloat16 if dtype == "bfloat16" else torch.float32
    spec = RoutedExpertsSpec(dim=D, n_experts=E, top=top, hidden=F_, n_groups=groups, keep_groups=keep,
                             shared_hidden=shared, activation="silu", scoring="sigmoid", choice_correction=True,
                             group_top=2, gated=True, shared_gate=bool(shared))
    part = FEED_FORWARDS.build(spec, Runtime(dt, DEV))
    w = {}
    for name, p in part.parameters().items():
        std = 0.6 if name == "w_router" else 0.15
        w[name] = (torch.randn(p.shape, generator=g) * std).to(dt if p.role == "matrix" else torch.float32)
    w["correction"] = torch.randn(E, generator=g) * 0.5 - 0.3
    part.bind({k: v.to(DEV) for k, v in w.items()})
    wd = {k: v.double() for k, v in w.items()}
    for n in (1, 2, 5, 16, 17, 40, 150):
        x = (torch.randn(n, D, generator=g) * 0.7).to(dt)
        xd = x.double()
        zd = xd @ wd["w_router"].T
        chosen, weights = P.route(zd, wd["correction"], top, groups, keep)
        want = torch.zeros(n, D, dtype=F)
        for e in range(E):
            weight = (weights * (chosen == e)).sum(-1, keepdim=True)
            want += weight * P.gated_expert(xd, wd["w_up"][e, :F_], wd["w_up"][e, F_:], wd["w_down"][e])
        if shared:
            want += torch.sigmoid(xd @ wd["shared_gate"].T) * P.gated_expert(
                xd, wd["shared_up"][:shared], wd["shared_up"][shared:], wd["shared_down"])
        for decode in (False, True):
            batch = types.SimpleNamespace(is_decode=decode)
            got = part.forward_rows(x.to(DEV), batch)
            if dtype == "float32":
                assert rel_err(got, want) < tol, (n, decode)
            else:
                assert float(row_errors(got, want).median()) < tol, (n, decode)
            assert (part.last_chosen.cpu().sort(-1).values == chosen.sort(-1).values).float().mean() > \
                (0.999 if dtype == "float32" else 0.9)


# --------------------------------------------------------------------------- whole models
@pytest.mark.parametrize("name", sorted(CASES))
@pytest.mark.parametrize("dtype,tol", [("float32", TOL_F32_LONG), ("bfloat16", TOL_BF16)])
def test_whole_prompt_at_every_position_and_the_stream_after_every_layer(tmp_path, name, dtype, tol):
    folder = make_folder(tmp_path, name, seed=11)
    cfg, w = P.load_folder(folder)
    toks = util.random_tokens(cfg["vocab"], 150, 3)
    outs = []
    want = P.forward(w, cfg, toks, outs)
    eng = _engine(folder, dtype)
    taps = []
    eng.model.tap = lambda n, x: taps.append(x.double().cpu())
    got = _steps(eng, toks, [])
    eng.model.tap = None
    assert close(got, want, dtype, tol)
    assert len(taps) == len(outs) == len(cfg["layers"])
    if dtype == "float32":
        for n, (a, b) in enumerate(zip(taps, outs)):
            assert rel_err(a, b) < TOL_F32_LONG, n
        # one token, and the first tokens of a sequence (fewer than the taps, than a window)
        assert rel_err(_steps(eng, toks[:1], []), want[:1]) < TOL_F32_LONG
        assert rel_err(_steps(eng, toks[:3], []), want[:3]) < TOL_F32_LONG
        assert rel_err(_steps(eng, toks[:3], [1, 2]), want[:3]) < TOL_F32_LONG


@pytest.mark.parametrize("name", sorted(CASES))
@pytest.mark.parametrize("dtype,tol", [("float32", TOL_F32_LONG), ("bfloat16", TOL_BF16)])
def test_portions_and_token_by_token_equal_the_whole_prompt(tmp_path, name, dtype, tol):
    folder = make_folder(tmp_path, name, seed=12)
    cfg, w = P.load_folder(folder)
    toks = util.random_tokens(cfg["vocab"], 210, 5)
    want = P.forward(w, cfg, toks)
    eng = _engine(folder, dtype)
    whole = _steps(eng, toks, [])
    assert close(whole, want, dtype, tol)
    for cuts in ([2, 4, 5, 70, 128, 129], [63, 64, 65, 192], [17, 150], list(range(150, 210)),
                 list(range(1, 80)), list(range(2, 210, 2))):
        got = _steps(eng, toks, cuts)
        assert close(got, want, dtype, tol), cuts
        assert close(got, whole, dtype, tol), cuts
    eng.cache.check()


@pytest.mark.parametrize("name", ["A", "B", "C"])
@pytest.mark.parametrize("dtype,same", [("float32", 2e-5), ("bfloat16", TOL_BF16)])
def test_unequal_batches_equal_each_request_alone(tmp_path, name, dtype, same):
    import gpt_fast_amd as gfa
    folder = make_folder(tmp_path, name, seed=13)
    cfg, w = P.load_folder(folder)
    lens = [1, 5, 131, 64, 70]
    tail = 30
    seqs = [util.random_tokens(cfg["vocab"], n + tail, 40 + n) for n in lens]
    eng = _engine(folder, dtype, max_tokens=64 * 20, max_sequences=6)
    alone = [_steps(eng, s, [n] + list(range(n + 1, n + tail))) for s, n in zip(seqs, lens)]
    slots = [eng.start_sequence() for _ in seqs]
    got = [[] for _ in seqs]
    out = eng.step([gfa.Entry(sl, s[:n], want=list(range(n))) for sl, s, n in zip(slots, seqs, lens)]).cpu()
    at = 0
    for b, n in enumerate(lens):
        got[b].append(out[at:at + n])
        at += n
    live = list(range(len(seqs)))
    for t in range(tail):
        if t == 10:                                  # a shorter request ends earlier
            eng.end_sequence(slots[1])
            live.remove(1)
        out = eng.step([gfa.Entry(slots[b], [seqs[b][lens[b] + t]], want=[0]) for b in live]).cpu()
        for i, b in enumerate(live):
            got[b].append(out[i:i + 1])
    for b in live:
        eng.end_sequence(slots[b])
    eng.cache.check()
    for b, s in enumerate(seqs):
        g = torch.cat(got[b])
        assert close(g, alone[b][:g.shape[0]], dtype, same), b
    want = P.forward(w, cfg, seqs[2])
    assert close(torch.cat(got[2]), want, dtype, TOL_F32_LONG)


@pytest.mark.parametrize("name", ["A", "C"])
@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_a_step_that_mixes_single_tokens_a_portion_and_a_new_prompt(tmp_path, name, dtype):
    import gpt_fast_amd as gfa
    folder = make_folder(tmp_path, name, seed=21)
    cfg, w = P.load_folder(folder)
    _, before, mixed = util.mixed_step_case(cfg["vocab"])
    lens = {"d0": 9, "d1": 66, "d2": 130, "c": 112, "p": 131}
    seqs = {r: util.random_tokens(cfg["vocab"], n, 300 + n) for r, n in lens.items()}
    eng = _engine(folder, dtype, max_tokens=64 * 16, max_sequences=5)
    slots = {r: eng.start_sequence() for r in seqs}
    got = {r: [] for r in seqs}
    order = ["d0", "d1", "d2", "c"]
    logits = eng.step([gfa.Entry(slots[r], seqs[r][:before[r]], want=list(range(before[r]))) for r in order]).cpu()
    at = 0
    for r in order:
        got[r].append(logits[at:at + before[r]])
        at += before[r]
    order = ["d0", "c", "d1", "p", "d2"]
    fed = {r: before.get(r, 0) for r in order}
    logits = eng.step([gfa.Entry(slots[r], seqs[r][fed[r]:fed[r] + mixed[r]], want=list(range(mixed[r])))
                       for r in order]).cpu()
    at = 0
    for r in order:
        got[r].append(logits[at:at + mixed[r]])
        at += mixed[r]
        fed[r] += mixed[r]
    for r in ("c", "p"):
        while fed[r] < len(seqs[r]):
            got[r].append(eng.step([gfa.Entry(slots[r], [seqs[r][fed[r]]], want=[0])]).cpu())
            fed[r] += 1
    for r in seqs:
        eng.end_sequence(slots[r])
    eng.cache.check()
    assert eng.cache.slots.held == 0
    for r, toks in seqs.items():
        g, want = torch.cat(got[r]), P.forward(w, cfg, toks)
        if dtype == "float32":
            assert rel_err(g, want) < TOL_F32_LONG, r
        else:
            assert close(g, _steps(eng, toks, []), dtype, TOL_F32_LONG), r
            assert float(row_errors(g, want).median()) < 2 * TOL_BF16, r


def test_slots_and_pages_that_come_back_start_clean(tmp_path):
    """A cache of few pages and two slots: requests follow one another in the same slots and
    pages (the delta rule's state and the convolutions' tails among their state, windows that
    give pages back while a request runs), and every request equals the plain computation of
    itself alone."""
    import gpt_fast_amd as gfa
    folder = make_folder(tmp_path, "A", seed=14)
    cfg, w = P.load_folder(folder)
    eng = _engine(folder, "float32", max_tokens=64 * 7, max_sequences=2)
    for round_ in range(3):
        a = util.random_tokens(cfg["vocab"], 150 + 90, 60 + round_)
        b = util.random_tokens(cfg["vocab"], 40 + 90, 70 + round_)
        sa, sb = eng.start_sequence(), eng.start_sequence()
        assert {sa, sb} == {0, 1}
        got_a, got_b = [], []
        out = eng.step([gfa.Entry(sa, a[:150], want=[149]), gfa.Entry(sb, b[:40], want=[39])]).cpu()
        got_a.append(out[0:1])
        got_b.append(out[1:2])
        for t in range(89):
            out = eng.step([gfa.Entry(sa, [a[150 + t]], want=[0]), gfa.Entry(sb, [b[40 + t]], want=[0])]).cpu()
            got_a.append(out[0:1])
            got_b.append(out[1:2])
        eng.cache.check()
        # a window of 40 and one of 70 keys: 240 tokens hold two pages per group, not four
        assert max(sum(p >= 0 for p in g.held[sa]) for _, g in eng.cache.paged_groups) <= 2
        eng.end_sequence(sb)
        eng.end_sequence(sa)
        assert rel_err(torch.cat(got_a), P.forward(w, cfg, a[:-1])[149:]) < TOL_F32_LONG
        assert rel_err(torch.cat(got_b), P.forward(w, cfg, b[:-1])[39:]) < TOL_F32_LONG
    for _, g in eng.cache.paged_groups:
        assert g.pages.held == 0


def test_state_that_lasts_hundreds_of_tokens_and_long_decoding(tmp_path):
    """Decays next to one in retention and in the delta rule: the first tokens decide the last
    logits five hundred tokens later, through a prompt and 130 tokens decoded one by one."""
    def patch(t):
        for name in t:
            if name.endswith(".A_log"):
                t[name] = torch.full_like(t[name], -7.0)
    config = dict(CASES["A"])
    config["layers"] = [dict(l) for l in config["layers"]]
    for l in config["layers"]:
        if l["type"] == "retention":
            l["mixer"] = dict(l["mixer"], decay=[0.999] * l["mixer"]["heads"])
    folder = write_model(os.path.join(str(tmp_path), "lasting"), config, 16, patch=patch)
    cfg, w = P.load_folder(folder)
    toks = util.random_tokens(cfg["vocab"], 520, 21)
    want = P.forward(w, cfg, toks)
    # it matters: with other first tokens the last logits are others
    other = util.random_tokens(cfg["vocab"], 20, 22) + toks[20:]
    assert rel_err(P.forward(w, cfg, other)[-40:], want[-40:]) > 1e-2
    for dtype in ("float32", "bfloat16"):
        eng = _engine(folder, dtype, max_tokens=64 * 10, max_sequences=1)
        got = _steps(eng, toks, [390] + list(range(391, 520)))
        if dtype == "float32":
            assert rel_err(got, want) < 3 * TOL_F32_LONG
        else:
            assert float(row_errors(got, want).median()) < TOL_BF16
        eng.cache.check()


@pytest.mark.parametrize("window", [1, 2, 37, 64, 65])
def test_a_window_s_edge_in_a_whole_model_in_prompts_and_in_decoding(tmp_path, window):
    """One layer whose attention alone carries information between tokens (the delta rule's
    output projection is zero): the logits at a position equal those of the same
    sequence with everything before the window replaced, and differ once the token just inside
    it is replaced; whole prompts and decoded tokens, against the plain implementation."""
    config = dict(CASES["A"])
    layer = dict(config["layers"][0])
    left = dict(layer["mixer"]["left"], mask={"size": window})
    layer["mixer"] = {"left": left, "right": layer["mixer"]["right"]}
    config["layers"] = [layer]

    def patch(t):
        t["l0.mix.right.o"] = torch.zeros_like(t["l0.mix.right.o"])
        t["l0.mix.left.q.norm"] = t["l0.mix.left.q.norm"] * 4
    folder = write_model(os.path.join(str(tmp_path), f"edge{window}"), config, 30 + window, patch=patch)
    cfg, w = P.load_folder(folder)
    T = 200
    toks = util.random_tokens(cfg["vocab"], T, 5)
    want = P.forward(w, cfg, toks)
    for at in (70, 128, 199):
        first_seen = at - window + 1
        if first_seen >= 1:
            outside = util.random_tokens(cfg["vocab"], first_seen, 6) + toks[first_seen:]
            assert rel_err(P.forward(w, cfg, outside)[at], want[at]) < 1e-9        # the oracle's own edge
        if window > 1:
            inside = list(toks)
            inside[first_seen] = (inside[first_seen] + 1) % cfg["vocab"]
            assert rel_err(P.forward(w, cfg, inside)[at], want[at]) > 1e-4
    for dtype, tol in (("float32", TOL_F32_LONG), ("bfloat16", TOL_BF16)):
        eng = _engine(folder, dtype, max_tokens=64 * 6, max_sequences=1)
        for cuts in ([], [60] + list(range(61, T)), [127, 129]):
            assert close(_steps(eng, toks, cuts), want, dtype, tol), (dtype, cuts)
        eng.cache.check()


@pytest.mark.parametrize("seed", [1, 2, 3, 4, 5, 6])
def test_random_configurations_whole_and_in_a_batch_that_is_decoded_together(tmp_path, seed):
    """Sizes drawn at random (refolix_cases.random_case): requests of 400, 130, 33 and 1 tokens,
    each whole, then their prompts in one batch and twenty tokens decoded together."""
    import gpt_fast_amd as gfa
    config = random_case(seed)
    folder = write_model(os.path.join(str(tmp_path), f"random{seed}"), config, 100 + seed, std=0.05)
    cfg, w = P.load_folder(folder)
    lens = [400, 130, 33, 1]
    seqs = [util.random_tokens(cfg["vocab"], n + 20, 7 * seed + n) for n in lens]
    want = [P.forward(w, cfg, s) for s in seqs]
    for dtype in ("float32", "bfloat16"):
        eng = _engine(folder, dtype, max_tokens=4096, max_sequences=4)

        def held(got, wanted):
            e = row_errors(got, wanted)
            if dtype == "float32":
                return float(e.max()) < 5e-4 and float(e.median()) < 3e-5
            # bfloat16: a router's close call falls the other way after the rounding of what the
            # router reads, and the rows behind it inherit the difference through the states; so
            # the typical row, and requests long enough for one
            if e.numel() < 100:
                return True
            return float(e.median()) < TOL_BF16

        for s, wanted in zip(seqs, want):
            assert held(_steps(eng, s, []), wanted), (dtype, len(s))
        slots = [eng.start_sequence() for _ in seqs]
        got = [[] for _ in seqs]
        out = eng.step([gfa.Entry(sl, s[:n], want=list(range(n))) for sl, s, n in zip(slots, seqs, lens)]).cpu()
        at = 0
        for b, n in enumerate(lens):
            got[b].append(out[at:at + n])
            at += n
        for t in range(20):
            out = eng.step([gfa.Entry(slots[b], [seqs[b][lens[b] + t]], want=[0]) for b in range(len(seqs))]).cpu()
            for b in range(len(seqs)):
                got[b].append(out[b:b + 1])
        for sl in slots:
            eng.end_sequence(sl)
        eng.cache.check()
        for b in range(len(seqs)):
            assert held(torch.cat(got[b]), want[b]), (dtype, b)


# --------------------------------------------------------------------------- generation
@pytest.mark.parametrize("name", ["A", "C"])
def test_greedy_generation_through_the_loop_and_the_recorded_step(tmp_path, name):
    from gpt_fast_amd.engine.generate import generate
    folder = make_folder(tmp_path, name, seed=17)
    cfg, w = P.load_folder(folder)
    prompts = [util.random_tokens(cfg["vocab"], n, 80 + n) for n in (7, 1, 90, 30)]
    want = [P.greedy_generate(w, cfg, p, 12) for p in prompts]
    eng = _engine(folder, "float32", max_tokens=64 * 12, max_sequences=4)
    assert eng.model.replayable
    for use_graph in (False, True, True):                       # the recording is replayed
        got = generate(eng, prompts, max_new_tokens=12, temperature=0.0, use_graph=use_graph)
        assert got.tokens == want, use_graph
    # two at a time: slots and state come back between the batches
    got = generate(eng, prompts, max_new_tokens=12, temperature=0.0, batch_size=2)
    assert got.tokens == want
    eng.cache.check()
    # bfloat16 through the recorded step: the tokens of the step that is not recorded
    eng = _engine(folder, "bfloat16", max_tokens=64 * 12, max_sequences=4)
    plain_steps = generate(eng, prompts, max_new_tokens=12, temperature=0.0, use_graph=False).tokens
    for _ in range(2):
        assert generate(eng, prompts, max_new_tokens=12, temperature=0.0, use_graph=True).tokens == plain_steps


def test_command_line_entry_point(tmp_path):
    import gpt_fast_amd as gfa
    folder = make_folder(tmp_path, "B", seed=18)
    cfg, w = P.load_folder(folder)
    prompt = util.random_tokens(cfg["vocab"], 20, 1)
    lines = []
    res = gfa.main(prompt=prompt, num_samples=1, max_new_tokens=8, temperature=0.0, top_k=None,
                   checkpoint_path=folder, dtype="float32", device=DEV, out=lines.append)
    assert res["result"].tokens[0] == P.greedy_generate(w, cfg, prompt, 8)
    assert any("tokens/sec" in str(l) for l in lines)


def test_trace_replay_program(tmp_path):
    """bin/trace_run as a program on a Refolix folder: two batches of unequal requests one after
    the other (the second takes the slots, state and pages the first gave back), logits wanted
    at some places only, steps in which nothing is wanted, a request that ends in the step that
    brings its prompt."""
    import json
    import subprocess

    import numpy as np
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    folder = make_folder(tmp_path, "C", seed=19)
    cfg, w = P.load_folder(folder)
    V = cfg["vocab"]
    reqs = {"a": util.random_tokens(V, 150, 1), "b": util.random_tokens(V, 9, 2), "c": util.random_tokens(V, 1, 3),
            "d": util.random_tokens(V, 200, 4), "e": util.random_tokens(V, 70, 5)}
    prompt = {"a": 120, "b": 3, "c": 1, "d": 130, "e": 64}
    steps, where = [], {r: [] for r in reqs}          # request -> (step, row in the file, position)
    n = 0
    for ids in (["a", "b", "c"], ["d", "e"]):
        live, t = list(ids), 0
        while live:
            entries, row = [], 0
            for r in live:
                lo, hi = (0, prompt[r]) if t == 0 else (prompt[r] + t - 1, prompt[r] + t)
                want = [i for i in range(hi - lo) if (lo + i) % 3 != 1]
                entries.append({"id": r, "tokens": reqs[r][lo:hi], "want": want})
                for i in want:
                    where[r].append((n, row, lo + i))
                    row += 1
            ends = [r for r in live if (prompt[r] + t if t else prompt[r]) >= len(reqs[r])]
            steps.append({"step": n, "entries": entries, "end": ends})
            live = [r for r in live if r not in ends]
            n += 1
            t += 1
    out_dir = os.path.join(str(tmp_path), "out")
    for dtype, tol in (("float32", TOL_F32_LONG), ("bfloat16", None)):
        proc = subprocess.run(
            [os.path.join(root, "bin", "trace_run"), "--model", folder, "--dtype", dtype, "--out", out_dir,
             "--max-tokens", "400"],
            input="".join(json.dumps(s) + "\n" for s in steps), capture_output=True, text=True, timeout=600)
        assert proc.returncode == 0, proc.stderr[-2000:]
        assert [l for l in proc.stdout.splitlines() if l.startswith("done ")] == [f"done {i}" for i in range(n)]
        for r, toks in reqs.items():
            want = P.forward(w, cfg, toks)
            got = torch.stack([torch.from_numpy(np.fromfile(os.path.join(out_dir, f"{s}.f32"), dtype="<f4")
                                                .reshape(-1, V)[row]) for s, row, _ in where[r]]) \
                if where[r] else torch.zeros(0, V)
            wanted = want[[p for _, _, p in where[r]]]
            if tol is not None:
                assert rel_err(got, wanted) < tol, r
            elif got.shape[0] >= 20:
                assert float(row_errors(got, wanted).median()) < TOL_BF16, r
