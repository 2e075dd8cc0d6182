"""Vusenex on the GPU against the plain float64 implementation of tests/plain_vusenex.py: each
mechanism's kernels alone (the pair embedding with its carried token, learned positions, the
gated and normed join, the whole-projection norm with its cache write, attention with a sink
and a bias by log distance, the latent without a query latent, the router and the experts'
products in each of their forms), whole prompts with the stream after every layer, prompts in
portions, token-by-token decoding, unequal batches, slots and pages that come back, far keys
and page borders with inputs that make one key stand out, long decoding, and greedy generation
through the library's generation loop, command line and trace replay."""
import math
import types

import pytest
import torch

import plain_vusenex as P
import util
from util import TOL_BF16, TOL_F32, rel_err
from vusenex_cases import CASES, make_folder

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
# float32 engine against float64 over a few hundred tokens and several normed joins
TOL_F32_LONG = 1e-4


def row_errors(got, want):
    """Per row: root mean square of the difference over that of all of ``want``."""
    got, want = got.double().cpu(), want.double().cpu()
    return (got - want).pow(2).mean(-1).sqrt() / want.pow(2).mean().sqrt()


def bf16_close(got, want):
    """A bfloat16 engine against float64: every sublayer's result is divided by its own root
    mean square before it joins the stream, and a router's close call may fall the other way
    after a rounding, so single rows can be off by more than the typical one.  The typical row
    is held to the tolerance and all but one in a hundred (at least one) to a bound that a
    wrong key, a lost state or a missing term, which touch most rows, would break.  The
    float32 engine is the sharp test."""
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


# --------------------------------------------------------------------------- the embedding's adds
@pytest.mark.parametrize("table_dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("buckets,mul_prev,mul_cur,dim", [(13, 7, 2, 40), (211, 31, 5, 96), (1, 3, 3, 50),
                                                         (262139, 1000003, 31, 64)])
def test_pair_embedding_rows_and_the_token_a_sequence_carries(table_dtype, buckets, mul_prev, mul_cur, dim):
    """Three sequences in slots 2, 0 and 3 of four; the second step goes on with two of them in
    another order, the third starts a new sequence in a slot that was used before."""
    from gpt_fast_amd.ops import kernels as K
    torch.manual_seed(buckets % 97)
    vocab = 100000 if buckets > 1000 else 50
    table = torch.randn(buckets + 1, dim).to(table_dtype).to(DEV)
    tbl = table.double().cpu()
    seqs = {2: util.random_tokens(vocab, 9, 1), 0: util.random_tokens(vocab, 4, 2), 3: util.random_tokens(vocab, 6, 3)}
    last = torch.full((4,), -7, dtype=torch.int32, device=DEV)
    fed = {s: 0 for s in seqs}

    def step(portions):
        slots = [s for s, _ in portions]
        lens = [n for _, n in portions]
        toks, pos, seq = [], [], []
        for b, (s, n) in enumerate(portions):
            toks += seqs[s][fed[s]:fed[s] + n]
            pos += list(range(fed[s], fed[s] + n))
            seq += [b] * n
        q_start = [sum(lens[:b]) for b in range(len(lens) + 1)]
        out = torch.randn(len(toks), dim, device=DEV)
        before = out.double().cpu()
        K.pair_embed_add(out, table, _ints(toks), _ints(seq), _ints(pos), _ints(q_start), _ints(slots),
                         last, buckets, mul_prev, mul_cur)
        at = 0
        for s, n in portions:
            rows = P.pair_rows(seqs[s][:fed[s] + n], buckets, mul_prev, mul_cur)[fed[s]:]
            assert rel_err(out[at:at + n].double().cpu() - before[at:at + n], tbl[rows]) < 1e-6, (s, fed[s])
            at += n
            fed[s] += n
            assert int(last[s]) == seqs[s][fed[s] - 1]

    step([(2, 5), (0, 1), (3, 2)])
    step([(3, 1), (2, 1)])
    step([(2, 3), (3, 3)])
    seqs[0], fed[0] = util.random_tokens(vocab, 5, 4), 0            # the slot comes back: position 0 again
    step([(0, 2)])
    step([(0, 1)])
    step([(0, 2)])


def test_learned_position_rows_are_added_unscaled():
    from gpt_fast_amd.ops import kernels as K
    torch.manual_seed(3)
    for dtype in (torch.float32, torch.bfloat16):
        table = torch.randn(70, 52).to(dtype).to(DEV)
        pos = [0, 1, 2, 69, 17, 17, 33]
        out = torch.randn(len(pos), 52, device=DEV)
        want = out.double().cpu() + table.double().cpu()[pos]
        K.add_table_rows(out, table, _ints(pos))
        assert rel_err(out, want) < 1e-6


# --------------------------------------------------------------------------- the gated, normed join
@pytest.mark.parametrize("dim", [50, 96, 1030, 4096, 8200])
def test_a_result_joins_the_stream_through_its_gate_and_its_norm(dim):
    from gpt_fast_amd.ops import kernels as K
    torch.manual_seed(dim)
    rows = 7
    res = torch.randn(rows, dim, device=DEV) * 2
    y = torch.randn(rows, dim, device=DEV) * 5
    wide = torch.randn(rows, dim + 8, device=DEV) * 3
    gate = wide[:, :dim]                                           # a view of wider rows
    bias = torch.randn(dim, device=DEV)
    g1 = torch.full((dim,), 0.7, device=DEV)
    w2 = torch.randn(dim, device=DEV)
    yy = y.double().cpu() * torch.sigmoid(gate.double().cpu() + bias.double().cpu())
    want = res.double().cpu() + P.scalar_norm(yy, torch.tensor(0.7, dtype=torch.float64), 1e-3)
    r = res.clone()
    assert K.gated_normed_add(r, y, g1, 1e-3, gate, bias) is None
    assert rel_err(r, want) < 1e-6
    # without a gate the result is only normed
    r0 = res.clone()
    K.gated_normed_add(r0, y, g1, 1e-3)
    assert rel_err(r0, res.double().cpu() + P.scalar_norm(y.double().cpu(), torch.tensor(0.7, dtype=torch.float64), 1e-3)) < 1e-6
    for dtype, tol in ((torch.float32, 1e-6), (torch.bfloat16, 1e-2)):
        r2 = res.clone()
        nxt = K.gated_normed_add(r2, y, g1, 1e-3, gate, bias, next_plain=True, out_dtype=dtype)
        assert torch.equal(r, r2) and nxt.dtype == dtype
        assert rel_err(nxt, want) < tol
        r3 = res.clone()
        nxt = K.gated_normed_add(r3, y, g1, 1e-3, gate, bias, next_weight=w2, next_eps=1e-6, out_dtype=dtype)
        assert torch.equal(r, r3)
        assert rel_err(nxt, P.unit_rms(want, 1e-6) * w2.double().cpu()) < tol


def test_exact_gelu_and_the_rows_of_the_stream_in_the_compute_type():
    from gpt_fast_amd.ops import kernels as K
    torch.manual_seed(4)
    x = torch.randn(7, 24, device=DEV) * 3
    x[0, :3] = torch.tensor([0.0, -20.0, 20.0])
    assert rel_err(K.activate(x, "gelu"), P.gelu_erf(x.double().cpu())) < 1e-6
    assert rel_err(K.activate(x.bfloat16(), "gelu"), P.gelu_erf(x.bfloat16().double().cpu())) < 1e-2
    assert torch.equal(K.cast_rows(x, torch.bfloat16), x.bfloat16())
    assert torch.equal(K.cast_rows(x, torch.float32, rows=_ints([6, 0, 0])), x[[6, 0, 0]])


# --------------------------------------------------------------------------- attention with a sink
@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-5), (torch.bfloat16, 1e-2)])
@pytest.mark.parametrize("H,G,d,coef,every", [(4, 2, 16, 0.5, 64), (3, 3, 20, 0.4, 16), (6, 1, 8, None, 1),
                                             (2, 1, 10, 1.5, 5), (8, 2, 64, 0.7, 1)])
def test_the_norm_over_the_whole_projection_the_temperature_and_the_cache(dtype, tol, H, G, d, coef, every):
    from gpt_fast_amd.ops import scored_attention as SA
    torch.manual_seed(H + d)
    lens, starts = [70, 1, 3], [0, 130, 62]
    n_pages, tables, table, tok_seq, tok_pos, pos = _table_and_positions(lens, starts)
    width = (H + G) * d
    proj = torch.randn(sum(lens), width + 3, device=DEV) * 2          # rows wider than what is read
    bias = torch.randn(width, device=DEV)
    qw, kw = 1 + 0.3 * torch.randn(H * d, device=DEV), 1 + 0.3 * torch.randn(G * d, device=DEV)
    k_pages = torch.zeros(n_pages, G, 64, d, device=DEV, dtype=dtype)
    v_pages = torch.zeros(n_pages, G, d, 64, device=DEV, dtype=dtype)
    q = SA.whole_norm_store(proj, bias, qw, kw, tok_seq, tok_pos, table, k_pages, v_pages, H, G, d, d,
                            1e-4, coef, every, True, dtype)
    x = proj[:, :width].double().cpu() + bias.double().cpu()
    want_q = P.unit_rms(x[:, :H * d], 1e-4) * qw.double().cpu()
    if coef is not None:
        temp = torch.tensor([1 + coef * math.log((p + 1) // every + 1) for p in pos], dtype=torch.float64)
        want_q = want_q * temp[:, None]
    want_k = (P.unit_rms(x[:, H * d:], 1e-4) * kw.double().cpu()).view(-1, G, d)
    want_v = x[:, H * d:].view(-1, G, d)                              # the keys as projected
    assert rel_err(q.view(-1, H * d), want_q) < tol
    k, v = _cache_rows(k_pages, v_pages, d, d)
    seqs = [b for b, l in enumerate(lens) for _ in range(l)]
    for n, (b, p_) in enumerate(zip(seqs, pos)):
        page = tables[b][p_ // 64]
        assert rel_err(k[page, :, p_ % 64], want_k[n]) < tol
        assert rel_err(v[page, :, :, p_ % 64], want_v[n]) < tol
    q2 = SA.whole_norm_store(proj, bias, qw, kw, tok_seq, tok_pos, table, None, None, H, G, d, d,
                             1e-4, coef, every, True, dtype)
    assert torch.equal(q, q2)


def _plain_sink_attention(q, k, v, start, scale, r1, r2, sink):
    """q [T, H, d] are the last T of the sequence's tokens; k [L, G, d], v [L, G, dv]."""
    T, H, _ = q.shape
    L, G, _ = k.shape
    i = torch.arange(T)[:, None] + start
    j = torch.arange(L)[None, :]
    see = j <= i
    dist = (i - j).clamp(min=0).double()
    out = []
    for h in range(H):
        s = (q[:, h] @ k[:, h // (H // G)].T) * scale
        if r1 is not None:
            s = s - r1[h] * torch.log1p(r2[h] * dist)
        if sink:
            a = P.sink_softmax(s, see)
        else:
            a = torch.softmax(s.masked_fill(~see, -math.inf), -1)
        out.append(a @ v[:, h // (H // G)])
    return torch.stack(out, 1)                                        # [T, H, dv]


def _attention_alone(dtype, H, G, d, dv, lens, starts, biased=True, sink=True, head_major=False,
                     boost=None, by_sequence=False, scale=0.4):
    """The attention kernel over sequences that already hold ``starts[b]`` tokens and get
    ``lens[b]`` more, pages handed out in reverse, against the plain attention.  ``boost``:
    (sequence, key position, factor) multiplies that key, so that its score stands out.
    ``by_sequence``: the step is also described sequence by sequence, which sends bfloat16 rows
    of sizes it takes to the matrix-core kernel."""
    from gpt_fast_amd.ops import scored_attention as SA
    torch.manual_seed(d * 7 + dv + H)
    total = [s + l for s, l in zip(starts, lens)]
    n_pages, tables, table, tok_seq, tok_pos, _ = _table_and_positions(lens, starts)
    ks = [torch.randn(t, G, d).to(dtype) for t in total]
    vs = [torch.randn(t, G, dv).to(dtype) for t in total]
    qs = [torch.randn(l, H, d).to(dtype) for l in lens]
    if boost is not None:
        b, key, factor = boost
        ks[b][key] *= factor
    # what lies beyond a sequence's end is not a number: a kernel that reads it spoils its sums
    k_rows = torch.full((n_pages, G, 64, d), float("nan"), dtype=dtype)
    v_cols = torch.full((n_pages, G, dv, 64), float("nan"), dtype=dtype)
    for b, t in enumerate(total):
        for pos in range(t):
            page = tables[b][pos // 64]
            k_rows[page, :, pos % 64] = ks[b][pos]
            v_cols[page, :, :, pos % 64] = vs[b][pos]
    k_pages = torch.empty_like(k_rows).view(n_pages, G, -1)
    v_pages = torch.empty_like(v_cols).view(n_pages, G, -1)
    k_pages[..., util.key_places(d).reshape(-1)] = k_rows.reshape(n_pages, G, -1)
    v_pages[..., util.value_places(dv).reshape(-1)] = v_cols.reshape(n_pages, G, -1)
    k_pages, v_pages = k_pages.view_as(k_rows).to(DEV), v_pages.view_as(v_cols).to(DEV)
    r1 = (torch.rand(H) * 1.5 + 0.1) if biased else None
    r2 = (torch.rand(H) * 0.5 + 0.02) if biased else None
    q = torch.cat(qs).to(DEV)
    q_in = q.permute(1, 0, 2).contiguous() if head_major else q
    step = None
    if by_sequence:
        step = (_ints([sum(lens[:b]) for b in range(len(lens) + 1)]), _ints(starts), len(lens), max(lens))
    out = SA.attention(q_in, k_pages, v_pages, tok_seq, tok_pos, table, scale,
                       log_bias=(r1.to(DEV), r2.to(DEV)) if biased else None, sink=sink,
                       head_major=head_major, step=step)
    if head_major:
        out = out.permute(1, 0, 2)
    at, worst = 0, 0.0
    for b, l in enumerate(lens):
        want = _plain_sink_attention(qs[b].double(), ks[b].double(), vs[b].double(), starts[b], scale,
                                     None if r1 is None else r1.double(), None if r2 is None else r2.double(), sink)
        got = out[at:at + l].double().cpu()
        assert not torch.isnan(got).any()
        worst = max(worst, rel_err(got, want))
        at += l
    return worst


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 2e-5), (torch.bfloat16, 2e-2)])
@pytest.mark.parametrize("H,G,d,biased,sink", [
    (4, 2, 16, True, True), (3, 3, 20, True, True), (6, 1, 8, True, True), (2, 1, 10, True, True),
    (4, 2, 64, True, True), (32, 8, 128, True, True), (6, 3, 16, False, True), (4, 2, 64, True, False),
    (1, 1, 12, True, True), (8, 1, 24, True, True), (12, 4, 32, True, True)])
@pytest.mark.parametrize("by_sequence", [False, True])
def test_attention_with_a_sink_and_a_bias_by_log_distance_alone(dtype, tol, H, G, d, biased, sink, by_sequence):
    """A prompt, a portion at an offset, single tokens and a first token, in one launch; on the
    plain kernel and (bfloat16, described sequence by sequence) on the matrix cores.  The
    values have the keys' size, as where the values are the keys."""
    if by_sequence and dtype != torch.bfloat16:
        pytest.skip("the matrix-core kernel is bfloat16 only")
    err = _attention_alone(dtype, H, G, d, d, lens=[130, 40, 1, 1, 3], starts=[0, 70, 200, 0, 63],
                           biased=biased, sink=sink, by_sequence=by_sequence)
    assert err < tol


def test_the_sink_takes_the_weight_that_no_key_earns():
    """Scores far below zero: with the sink the result shrinks towards nothing, without it the
    softmax still sums to one; scores far above zero: the sink does not matter."""
    for dtype, tol in ((torch.float32, 2e-5), (torch.bfloat16, 2e-2)):
        for by_sequence in (False, True):
            for scale in (-3.0, 3.0):
                err = _attention_alone(dtype, 4, 2, 16, 16, [90, 1], [0, 130], biased=False, sink=True,
                                       by_sequence=by_sequence, scale=scale)
                assert err < tol


@pytest.mark.parametrize("single", [1, 6])
def test_single_token_steps_of_attention_with_a_sink(single):
    """One token per sequence: sequences of one key, of less than a block, of several pages."""
    starts = [0, 5, 31, 32, 200, 700][:single]
    for H, G, d in ((4, 2, 64), (8, 8, 128), (6, 3, 16), (32, 8, 128)):
        err = _attention_alone(torch.bfloat16, H, G, d, d, lens=[1] * single, starts=starts, by_sequence=True)
        assert err < 2e-2
        err = _attention_alone(torch.float32, H, G, d, d, lens=[1] * single, starts=starts)
        assert err < 2e-5


@pytest.mark.parametrize("key", [0, 1, 63, 64, 65, 127, 128, 300, 448, 449])
def test_a_far_key_among_hundreds_stands_out(key):
    """One key far back, at a page's border, the first, the last, is multiplied by 12 and takes
    the softmax in spite of the bias by its distance; in a prompt, in a portion of two tokens
    and in a single-token step, on both kernels."""
    for lens, starts in (([450], [0]), ([2], [448]), ([1], [449])):
        err = _attention_alone(torch.float32, 4, 2, 16, 16, lens, starts, boost=(0, key, 12.0))
        assert err < 2e-5
        err = _attention_alone(torch.bfloat16, 4, 2, 16, 16, lens, starts, boost=(0, key, 12.0), by_sequence=True)
        assert err < 2e-2


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-5), (torch.bfloat16, 1e-2)])
@pytest.mark.parametrize("H,d,R", [(3, 16, 32), (2, 12, 20), (4, 8, 144), (2, 10, 14), (1, 20, 28)])
def test_the_latent_without_a_query_latent_and_without_a_rotated_part(dtype, tol, H, d, R):
    """The joined projection's rows are [kv latent | q]: the latent is normed and stored as key
    and as value, q leaves the kernel head by head; then ordinary softmax attention over the
    latents with one kv head."""
    from gpt_fast_amd.ops import scored_attention as SA
    torch.manual_seed(R + d)
    lens, starts = [70, 1, 3], [0, 130, 62]
    n_pages, tables, table, tok_seq, tok_pos, pos = _table_and_positions(lens, starts)
    N = sum(lens)
    proj = torch.randn(N, R + H * d + 5, device=DEV) * 2
    wkv = 1 + 0.3 * torch.randn(R, device=DEV)
    k_pages = torch.zeros(n_pages, 1, 64, R, device=DEV, dtype=dtype)
    v_pages = torch.zeros(n_pages, 1, R, 64, device=DEV, dtype=dtype)
    SA.latent_store(proj, 0, R, 0, None, wkv, 1e-4, None, 0, tok_seq, tok_pos, table, k_pages, v_pages, dtype)
    x = proj.double().cpu()
    want_c = P.unit_rms(x[:, :R], 1e-4) * wkv.double().cpu()
    k, v = _cache_rows(k_pages, v_pages, R, R)
    seqs = [b for b, l in enumerate(lens) for _ in range(l)]
    for n, (b, p_) in enumerate(zip(seqs, pos)):
        page = tables[b][p_ // 64]
        assert rel_err(k[page, 0, p_ % 64], want_c[n]) < tol
        assert rel_err(v[page, 0, :, p_ % 64], want_c[n]) < tol
    q = proj[:, R:R + H * d]                                          # a view of the wider rows
    plain, full = SA.latent_query(q, None, 0, tok_pos, H, d, 0, R, dtype)
    assert rel_err(plain.permute(1, 0, 2), q.double().cpu().view(N, H, d)) < tol
    assert tuple(full.shape) == (H, N, R)
    for by_sequence in (False, True):
        if by_sequence and dtype != torch.bfloat16:
            continue
        err = _attention_alone(dtype, H, 1, R, R, lens=[130, 40, 1, 1, 3], starts=[0, 70, 200, 0, 63],
                               biased=False, sink=False, head_major=True, by_sequence=by_sequence)
        assert err < 2 * tol


# --------------------------------------------------------------------------- the mixture of experts
@pytest.mark.parametrize("E,top,groups,keep", [(6, 2, 3, 2), (4, 1, 2, 1), (8, 3, 4, 2), (5, 2, 1, 1), (3, 3, 1, 1),
                                               (64, 6, 8, 3), (6, 2, 6, 3), (130, 5, 10, 4), (8, 3, 2, 1), (2, 1, 2, 2)])
def test_the_router_keeps_groups_then_takes_the_top(E, top, groups, keep):
    from gpt_fast_amd.ops import routed_experts as RE
    torch.manual_seed(E * 10 + top)
    wide = torch.randn(90, E + 3, device=DEV) * 2
    z = wide[:, :E]
    chosen, weights = RE.route(z, E, top, groups, keep, 1e-20)
    want = P.route(z.double().cpu(), top, groups, keep)               # [N, E] weights
    got = torch.zeros(90, E, dtype=torch.float64)
    got.scatter_(1, chosen.long().cpu(), weights.double().cpu())
    assert rel_err(got, want) < 1e-5
    assert bool((got > 0).sum(-1).eq(top).all())
    # in the order of falling scores
    assert bool((weights[:, :-1] >= weights[:, 1:]).all())
    assert rel_err(weights.sum(-1), torch.ones(90)) < 1e-5


def test_the_router_by_hand():
    from gpt_fast_amd.ops import routed_experts as RE
    # six experts in three groups; group maxima 0.05, 0.30, 0.28: groups 1 and 2 are kept
    z = torch.log(torch.tensor([[0.05, 0.04, 0.30, 0.01, 0.28, 0.27]])).to(DEV)
    chosen, weights = RE.route(z, 6, 2, 3, 2, 1e-20)
    assert chosen.cpu().tolist() == [[2, 4]]
    s = torch.softmax(z.double().cpu(), -1)[0]
    assert rel_err(weights, (s[[2, 4]] / (s[2] + s[4]))[None]) < 1e-6
    # with one kept group the second-largest expert overall cannot be chosen
    chosen, _ = RE.route(z, 6, 2, 3, 1, 1e-20)
    assert chosen.cpu().tolist() == [[2, 3]]
    chosen, weights = RE.route(z, 6, 1, 1, 1, 1e-20)
    assert chosen.cpu().tolist() == [[2]] and abs(float(weights[0, 0]) - 1) < 1e-6


def _dense_experts(x, wu, wd, chosen, weights, round_h):
    """Every pair by itself in float64; ``round_h``: the inner rows are rounded to bfloat16 as
    the bfloat16 kernels store them."""
    n, top = chosen.shape
    want = torch.zeros(n, wd.shape[1], dtype=torch.float64)
    xc, wuc, wdc = x.double().cpu(), wu.double().cpu(), wd.double().cpu()
    for i in range(n):
        for k in range(top):
            e = int(chosen[i, k])
            h = P.gelu_erf(wuc[e] @ xc[i])
            if round_h:
                h = h.bfloat16().double()
            want[i] += float(weights[i, k]) * (wdc[e] @ h)
    return want


@pytest.mark.parametrize("n,E,top,D,F_", [(1, 4, 2, 64, 40), (8, 6, 2, 96, 40), (5, 8, 3, 104, 24), (40, 4, 4, 72, 136),
                                         (64, 32, 4, 256, 64), (130, 3, 2, 64, 48), (3, 5, 2, 100, 18), (17, 4, 1, 50, 22)])
def test_the_experts_products_pair_by_pair_expert_by_expert_and_in_sorted_order(n, E, top, D, F_):
    """The same pairs through the forms the products take: one pair at a time (float32 and
    bfloat16) and expert by expert on the matrix cores (bfloat16, rows that are multiples of
    eight); the pairs' order by expert, their gathered rows (also with every expert's share
    padded to the largest) and the sum through the pairs' places."""
    from gpt_fast_amd.ops import routed_experts as RE
    torch.manual_seed(n + E)
    z = torch.randn(n, E, device=DEV)
    chosen, weights = RE.route(z, E, top, 1, 1, 1e-20)
    for dtype, tol in ((torch.float32, 1e-5), (torch.bfloat16, 1e-2)):
        x = torch.randn(n, D, device=DEV).to(dtype)
        wu = (torch.randn(E, F_, D, device=DEV) * 0.2).to(dtype)
        wd = (torch.randn(E, D, F_, device=DEV) * 0.2).to(dtype)
        want = _dense_experts(x, wu, wd, chosen, weights, dtype == torch.bfloat16)
        assert rel_err(RE.experts_few_rows(x, wu, wd, chosen, weights, "gelu"), want) < tol
        start = torch.randn(n, D, device=DEV)
        got = RE.experts_few_rows(x, wu, wd, chosen, weights, "gelu", out=start.clone())
        assert rel_err(got.double().cpu() - start.double().cpu(), want) < max(tol, 1e-4)
        offsets, order, place = RE.expert_order(chosen, E)
        counts = torch.bincount(chosen.flatten().long().cpu(), minlength=E)
        assert offsets.cpu().tolist() == [0] + counts.cumsum(0).tolist()
        assert sorted(order.cpu().tolist()) == list(range(n * top))
        assert torch.equal(order[place.long()].cpu(), torch.arange(n * top, dtype=torch.int32))
        e_sorted = chosen.flatten()[order.long()].cpu().tolist()
        assert e_sorted == sorted(e_sorted)
        xs = RE.gather_pairs(x, order, top)
        assert torch.equal(xs, x[(order // top).long()])
        cap = (int(counts.max()) + 7) // 8 * 8
        padded = RE.gather_pairs_padded(x, order, offsets, top, E, cap)
        where = RE.padded_places(place, chosen, offsets, cap)
        assert tuple(padded.shape) == (E, cap, D)
        assert torch.equal(padded.view(E * cap, D)[where.long()], x[(torch.arange(n * top, device=DEV) // top)])
        for e in range(E):
            assert float(padded[e, int(counts[e]):].abs().max() if int(counts[e]) < cap else 0.0) == 0.0
        direct = RE.combine_pairs(xs.float(), place, weights)
        assert torch.equal(RE.combine_pairs(padded.view(E * cap, D).float(), where, weights), direct)
        if dtype == torch.bfloat16 and D % 8 == 0 and F_ % 8 == 0:
            assert RE.grouped_rows_take(x, wu)
            h = RE.grouped_rows(x, order, top, wu, offsets, "gelu", n)
            ys = RE.grouped_rows(h, None, 1, wd, offsets, None, n)
            assert h.dtype == torch.bfloat16 and ys.dtype == torch.float32
            assert rel_err(RE.combine_pairs(ys, place, weights), want) < tol
            got = RE.combine_pairs(ys, place, weights, out=start.clone())
            assert rel_err(got.double().cpu() - start.double().cpu(), want) < tol
        elif dtype == torch.bfloat16:
            assert not (RE.grouped_rows_take(x, wu) and F_ % 8 == 0)


def test_a_pairs_result_does_not_depend_on_the_other_pairs():
    """Expert by expert on the matrix cores: a token alone, and the same token among 63 others
    that choose the same experts, bit for bit."""
    from gpt_fast_amd.ops import routed_experts as RE
    torch.manual_seed(9)
    n, E, top, D, F_ = 64, 4, 2, 128, 72
    x = torch.randn(n, D, device=DEV).bfloat16()
    wu = (torch.randn(E, F_, D, device=DEV) * 0.2).bfloat16()
    wd = (torch.randn(E, D, F_, device=DEV) * 0.2).bfloat16()
    chosen, weights = RE.route(torch.randn(n, E, device=DEV), E, top, 1, 1, 1e-20)

    def run(rows):
        c, w = chosen[rows].contiguous(), weights[rows].contiguous()
        offsets, order, place = RE.expert_order(c, E)
        h = RE.grouped_rows(x[rows].contiguous(), order, top, wu, offsets, "gelu", len(rows))
        return RE.combine_pairs(RE.grouped_rows(h, None, 1, wd, offsets, None, len(rows)), place, w)

    together = run(list(range(n)))
    for i in (0, 17, 63):
        assert torch.equal(run([i])[0], together[i])


@pytest.mark.parametrize("dtype,tol", [("float32", 1e-5), ("bfloat16", 2e-2)])
@pytest.mark.parametrize("D,E,top,groups,keep,F_,shared", [(72, 6, 2, 3, 2, 40, 56), (104, 4, 1, 2, 1, 24, 0),
                                                          (64, 8, 3, 4, 2, 16, 8), (100, 3, 3, 1, 1, 18, 10)])
def test_the_mixture_part_alone_at_every_number_of_rows(dtype, tol, D, E, top, groups, keep, F_, shared):
    """The part against the plain mixture: one row, few rows, the sizes at which it changes its
    way (16 and 17), many rows, and many single-token rows of a decoding step."""
    from gpt_fast_amd.config.spec import RoutedExpertsSpec
    from gpt_fast_amd.parts.base import FEED_FORWARDS, Runtime
    rt = Runtime(torch.float32 if dtype == "float32" else torch.bfloat16, DEV)
    torch.manual_seed(D + E)
    part = FEED_FORWARDS.build(RoutedExpertsSpec(dim=D, n_experts=E, top=top, hidden=F_, n_groups=groups,
                                                 keep_groups=keep, shared_hidden=shared, activation="gelu"), rt)
    t = {"w_router": (torch.randn(E, D, device=DEV) * 0.6).to(rt.dtype),
         "w_up": (torch.randn(E, F_, D, device=DEV) * 0.2).to(rt.dtype),
         "w_down": (torch.randn(E, D, F_, device=DEV) * 0.2).to(rt.dtype)}
    if shared:
        t["shared_up"] = (torch.randn(shared, D, device=DEV) * 0.2).to(rt.dtype)
        t["shared_down"] = (torch.randn(D, shared, device=DEV) * 0.2).to(rt.dtype)
    assert sorted(part.parameters()) == sorted(t)
    part.bind(dict(t))
    w = {"m.router": t["w_router"].double().cpu()}
    for e in range(E):
        w[f"m.e{e}.up"], w[f"m.e{e}.down"] = t["w_up"][e].double().cpu(), t["w_down"][e].double().cpu()
    if shared:
        w["m.shared.up"], w["m.shared.down"] = t["shared_up"].double().cpu(), t["shared_down"].double().cpu()
    mlp = {"router": {"experts": E, "top": top, "groups": {"count": groups, "keep": keep}},
           "shared": {"ff": shared} if shared else None}
    for rows, decode, skew in ((1, True, 0), (5, False, 0), (16, False, 0), (17, False, 0), (150, False, 0),
                               (40, True, 0), (150, False, 6.0)):
        x = torch.randn(rows, D, device=DEV).to(rt.dtype)
        if skew:
            # most tokens choose the same experts: shares too unequal for the padded product
            x = (x.float() + skew * t["w_router"][0].float() / t["w_router"][0].float().norm() * D ** 0.5).to(rt.dtype)
        want = P.mixture(x.double().cpu(), w, "m.", mlp)
        batch = types.SimpleNamespace(is_decode=decode)
        got = part.forward_rows(x, batch)
        assert got.dtype == torch.float32
        if dtype == "float32":
            assert rel_err(got, want) < tol, rows
        else:
            # a router's close call may fall the other way after the rounding of its sums' inputs
            assert float(row_errors(got, want).median()) < tol, rows
        res = torch.randn(rows, D, device=DEV)
        before = res.clone()
        part.forward(x, batch, res)
        assert rel_err(res - before, got) < 1e-5


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
        # one token, and the first tokens of a sequence
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
                 list(range(1, 80))):
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
    pages (the carried token of the pair embedding among their state), and every request
    equals the plain computation of itself alone."""
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
        eng.end_sequence(sb)
        eng.end_sequence(sa)
        assert rel_err(torch.cat(got_a), P.forward(w, cfg, a[:-1])[149:]) < TOL_F32_LONG
        assert rel_err(torch.cat(got_b), P.forward(w, cfg, b[:-1])[39:]) < TOL_F32_LONG
    for _, g in eng.cache.kv_groups:
        assert g.pages.held == 0


def test_peaked_softmax_over_a_long_prompt_and_long_decoding(tmp_path):
    """Queries scaled up until a head's weight sits on one or two keys among some hundred
    candidates, and the distance bias's numbers made large in half of the heads so that the
    far keys fall behind the sink; then 130 tokens decoded one by one across page borders."""
    def patch(t):
        for name in t:
            if name.endswith("mix.q.norm") or (name.endswith("mix.q") and name.replace("mix.q", "mix.dkv") in t):
                t[name] = t[name] * 5
            if name.endswith("mix.r1"):
                t[name][::2] = t[name][::2] * 4
    for name in ("A", "C"):
        folder = make_folder(tmp_path, name, seed=16, patch=patch, tag="peaked")
        cfg, w = P.load_folder(folder)
        toks = util.random_tokens(cfg["vocab"], 400, 21)
        want = P.forward(w, cfg, toks)
        # it matters: without the first 200 tokens the last logits are others
        assert rel_err(P.forward(w, cfg, toks[200:])[-40:], want[-40:]) > 1e-2
        for dtype in ("float32", "bfloat16"):
            eng = _engine(folder, dtype, max_tokens=64 * 8, max_sequences=1)
            got = _steps(eng, toks, [270] + list(range(271, 400)))
            if dtype == "float32":
                assert rel_err(got, want) < TOL_F32_LONG
            else:
                assert float(row_errors(got, want).median()) < TOL_BF16
            eng.cache.check()


@pytest.mark.parametrize("seed", [1, 2, 3, 4, 5, 6, 7, 8])
def test_random_configurations_whole_and_in_a_batch_that_is_decoded_together(tmp_path, seed):
    """Sizes drawn at random (vusenex_cases.random_case): requests of 700, 130, 33 and 1 tokens,
    each whole, then their prompts in one batch and twenty tokens decoded together."""
    import gpt_fast_amd as gfa
    import os
    from vusenex_cases import random_case, write_model
    config = random_case(seed)
    folder = write_model(os.path.join(str(tmp_path), f"random{seed}"), config, 100 + seed, std=0.05)
    cfg, w = P.load_folder(folder)
    lens = [700, 130, 33, 1]
    seqs = [util.random_tokens(cfg["vocab"], n + 20, 7 * seed + n) for n in lens]
    want = [P.forward(w, cfg, s) for s in seqs]
    for dtype in ("float32", "bfloat16"):
        eng = _engine(folder, dtype, max_tokens=4096, max_sequences=4)

        def held(got, wanted):
            e = row_errors(got, wanted)
            if dtype == "float32":
                # scores of several tens carry their float32 rounding into the softmax: a row
                # may be ten times the typical one
                return float(e.max()) < 5e-4 and float(e.median()) < 2e-5
            # bfloat16: a router's close call (0.48 against 0.52 in one of these) falls the other
            # way after the rounding of what the router reads, and the rows behind it inherit the
            # difference through attention; so the typical row, and requests long enough for one
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


def test_positions_beyond_the_learned_table_are_refused(tmp_path):
    import gpt_fast_amd as gfa
    folder = make_folder(tmp_path, "O", seed=20)
    cfg, _ = P.load_folder(folder)
    eng = _engine(folder, "float32", max_tokens=64 * 12, max_sequences=1)
    toks = util.random_tokens(cfg["vocab"], cfg["max_positions"] + 1, 2)
    slot = eng.start_sequence()
    with pytest.raises(Exception):
        eng.step([gfa.Entry(slot, toks, want=[0])])


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
    """bin/trace_run as a program on a Vusenex folder: two batches of unequal requests one after
    the other (the second takes the slots, state and pages the first gave back), logits wanted
    at some places only, steps in which nothing is wanted, a request that ends in the step that
    brings its prompt."""
    import json
    import os
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
            ending = [r for r in live if prompt[r] + t >= len(reqs[r])]
            steps.append({"step": n, "entries": entries, "end": ending})
            live = [r for r in live if r not in ending]
            n += 1
            t += 1
    lines = "\n".join(json.dumps(s) for s in steps) + "\n"
    for dtype in ("float32", "bfloat16"):
        out = str(tmp_path / dtype)
        proc = subprocess.run([os.path.join(root, "bin", "trace_run"), "--model", folder, "--dtype", dtype,
                               "--out", out, "--max-tokens", str(200 + 70)],
                              input=lines, capture_output=True, text=True, timeout=110)
        assert proc.returncode == 0, proc.stderr[-2000:]
        assert [l for l in proc.stdout.splitlines() if l.startswith("done")] == [f"done {s['step']}" for s in steps]
        for r, toks in reqs.items():
            want = P.forward(w, cfg, toks)
            rows, places = [], []
            for step, row, pos in where[r]:
                data = np.fromfile(os.path.join(out, f"{step}.f32"), dtype="<f4").reshape(-1, V)
                rows.append(torch.from_numpy(data[row].copy()))
                places.append(pos)
            assert close(torch.stack(rows), want[places], dtype, TOL_F32_LONG), (dtype, r)
        for s in steps:
            if not any(e["want"] for e in s["entries"]):
                assert not os.path.exists(os.path.join(out, f"{s['step']}.f32"))
