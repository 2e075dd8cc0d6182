"""CPU tests of Refolix: what fixes the plain implementation of tests/plain_refolix.py beside its
equations (hand-made cases and identities of each mechanism), the configuration reader, the
checkpoint layout against the model's parameters, the rescaled frequency ladder, and the joint
cache need's bookkeeping."""
import copy
import math

import pytest
import torch

import plain_refolix as P
import util
from refolix_cases import CASES, make_folder, random_case

F = torch.float64


# --------------------------------------------------------------------------- the plain implementation
def test_layer_norm_has_zero_mean_unit_variance_and_eps_inside_the_root():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(5, 40, generator=g, dtype=F) * 3 + 2
    w = torch.rand(40, generator=g, dtype=F) + 0.5
    y = P.layer_norm(x, torch.ones(40, dtype=F), 0.0)
    assert float(y.mean(-1).abs().max()) < 1e-12 and float((y.var(-1, unbiased=False) - 1).abs().max()) < 1e-12
    want = torch.nn.functional.layer_norm(x, (40,), w, None, 1e-3)
    assert util.rel_err(P.layer_norm(x, w, 1e-3), want) < 1e-12
    # a row of equal numbers: the deviations are zero, eps keeps the root from zero
    assert float(P.layer_norm(torch.full((1, 8), 7.0, dtype=F), torch.ones(8, dtype=F), 1e-6).abs().max()) == 0.0
    # the sum's scale does not matter (but for eps): what the stream's factor changes is the mix
    assert util.rel_err(P.layer_norm(5 * x, w, 0.0), P.layer_norm(x, w, 0.0)) < 1e-12


@pytest.mark.parametrize("layout", ["interleaved", "half"])
def test_rotation_pairs_sign_and_relative_positions(layout):
    rot = {"dims": 6, "base": 50.0}
    x = torch.zeros(1, 1, 8, dtype=F)
    first, second = (0, 1) if layout == "interleaved" else (0, 3)
    x[0, 0, first] = 1.0
    y = P.rotate(x, torch.tensor([2]), rot, layout)
    # pair 0 turns by 2 * f_0 = 2 radians: (1, 0) -> (cos 2, sin 2); the rest stays
    assert abs(float(y[0, 0, first]) - math.cos(2.0)) < 1e-12 and abs(float(y[0, 0, second]) - math.sin(2.0)) < 1e-12
    assert float(y[0, 0].abs().sum()) == pytest.approx(abs(math.cos(2.0)) + abs(math.sin(2.0)))
    g = torch.Generator().manual_seed(1)
    q, k = torch.randn(1, 1, 8, generator=g, dtype=F), torch.randn(1, 1, 8, generator=g, dtype=F)
    # elements behind the rotated ones pass unchanged; position 0 is the identity
    assert torch.equal(P.rotate(q, torch.tensor([9]), rot, layout)[..., 6:], q[..., 6:])
    assert util.rel_err(P.rotate(q, torch.tensor([0]), rot, layout), q) < 1e-15

    def dot(i, j):
        return float((P.rotate(q, torch.tensor([i]), rot, layout) * P.rotate(k, torch.tensor([j]), rot, layout)).sum())
    assert dot(17, 11) == pytest.approx(dot(106, 100), abs=1e-10)
    assert abs(dot(17, 11) - dot(17, 12)) > 1e-3


def test_the_rescaled_ladder_by_hand():
    """dims 8, base 100, original 64, factor 4, fast 16, slow 2: place(t) = 8 ln(64 / (2 pi t)) /
    (2 ln 100); place(16) = -0.39 -> lo 0; place(2) = 1.41 -> hi 2; ramp = 0, 1/2, 1, 1."""
    rot = {"dims": 8, "base": 100.0, "scaling": {"factor": 4.0, "original": 64, "fast": 16.0, "slow": 2.0}}
    f, grow = P.rotary_frequencies(rot)
    plain = [100.0 ** (-2.0 * i / 8) for i in range(4)]
    want = [plain[0], plain[1] * (0.5 / 4 + 0.5), plain[2] / 4, plain[3] / 4]
    assert util.rel_err(f, torch.tensor(want, dtype=F)) < 1e-12
    assert grow == pytest.approx(0.1 * math.log(4.0) + 1.0)
    # the library's ladder is the same one
    from gpt_fast_amd.config.spec import PositionSpec
    from gpt_fast_amd.parts.position import frequencies_and_trig_scale
    spec = PositionSpec(rotary_dim=8, base=100.0, layout="interleaved",
                        scaling=(("rope_type", "yarn"), ("factor", 4.0), ("original", 64), ("fast", 16.0), ("slow", 2.0)))
    freqs, trig = frequencies_and_trig_scale(spec)
    assert util.rel_err(freqs, f) < 1e-6 and trig == pytest.approx(grow)
    # without a rule: the plain ladder and no factor
    freqs, trig = frequencies_and_trig_scale(PositionSpec(rotary_dim=8, base=100.0))
    assert util.rel_err(freqs, torch.tensor(plain)) < 1e-6 and trig == 1.0
    # hi = lo: the ramp is a step (its width is held at 0.001)
    rot["scaling"].update(fast=2.0, slow=2.0)
    f, _ = P.rotary_frequencies(rot)          # place(2) = 1.41: lo = 1, hi = 2
    assert util.rel_err(f, torch.tensor([plain[0], plain[1], plain[2] / 4, plain[3] / 4], dtype=F)) < 1e-12


def test_window_mask_and_attention_see_exactly_the_window():
    m = P.window_mask(6, 3)
    assert m[5].tolist() == [False, False, False, True, True, True]
    assert m[1].tolist() == [True, True, False, False, False, False]
    assert P.window_mask(4, None)[3].tolist() == [True] * 4
    assert P.window_mask(4, 1)[2].tolist() == [False, False, True, False]


def test_short_convolution_against_the_library_s_convolution_and_by_hand():
    g = torch.Generator().manual_seed(2)
    x, taps = torch.randn(9, 5, generator=g, dtype=F), torch.randn(5, 4, generator=g, dtype=F)
    want = torch.nn.functional.conv1d(torch.nn.functional.pad(x.T[None], (3, 0)), taps[:, None, :], groups=5)[0].T
    assert util.rel_err(P.short_convolution(x, taps), want) < 1e-12
    # the last column weighs the current token; the first token sees zeros before it
    y = P.short_convolution(torch.tensor([[1.0], [10.0], [100.0]], dtype=F), torch.tensor([[3.0, 2.0]], dtype=F))
    assert y[:, 0].tolist() == [2.0, 23.0, 230.0]
    # one tap: a factor per channel
    assert util.rel_err(P.short_convolution(x, taps[:, :1]), x * taps[:, 0]) < 1e-15


def _tiny_delta(T, H, G, d, dv, seed):
    g = torch.Generator().manual_seed(seed)
    D = 12
    m = {"heads": H, "kv_heads": G, "dim": d, "vdim": dv, "conv": 2}
    w = {"q": torch.randn(G * d, D, generator=g, dtype=F), "k": torch.randn(G * d, D, generator=g, dtype=F),
         "v": torch.randn(H * dv, D, generator=g, dtype=F), "b": torch.randn(H, D, generator=g, dtype=F),
         "a": torch.randn(H, D, generator=g, dtype=F), "g": torch.randn(H * dv, D, generator=g, dtype=F),
         "o": torch.randn(D, H * dv, generator=g, dtype=F), "A_log": torch.randn(H, generator=g, dtype=F) - 1,
         "dt_bias": torch.randn(H, generator=g, dtype=F), "norm": torch.rand(dv, generator=g, dtype=F) + 0.5,
         "q.conv": torch.randn(G * d, 2, generator=g, dtype=F), "k.conv": torch.randn(G * d, 2, generator=g, dtype=F),
         "v.conv": torch.randn(H * dv, 2, generator=g, dtype=F)}
    return m, {"x." + k: v for k, v in w.items()}, torch.randn(T, D, generator=g, dtype=F)


def test_the_delta_rule_is_causal_and_its_state_has_the_closed_form():
    m, w, h = _tiny_delta(12, 4, 2, 6, 5, 3)
    whole = P.delta_rule(h, w, "x.", m, 1e-5)
    # a later token changes nothing earlier
    h2 = h.clone()
    h2[9] += 1.0
    assert util.rel_err(P.delta_rule(h2, w, "x.", m, 1e-5)[:9], whole[:9]) < 1e-12
    assert util.rel_err(P.delta_rule(h2, w, "x.", m, 1e-5)[9:], whole[9:]) > 1e-6
    # S <- g S; u = beta (v - S^T k); S <- S + k u^T   is   S <- g (I - beta k k^T) S + beta k v^T
    g = torch.Generator().manual_seed(5)
    S = torch.randn(6, 5, generator=g, dtype=F)
    k = torch.randn(6, generator=g, dtype=F)
    k = k / k.norm()
    v, beta, gate = torch.randn(5, generator=g, dtype=F), 0.7, 0.9
    S1 = gate * S
    S1 = S1 + torch.outer(k, beta * (v - S1.T @ k))
    S2 = gate * (torch.eye(6, dtype=F) - beta * torch.outer(k, k)) @ S + beta * torch.outer(k, v)
    assert util.rel_err(S1, S2) < 1e-12
    # with beta = 1 the state answers the key it has just been given with that value
    S3 = S + torch.outer(k, v - S.T @ k)
    assert util.rel_err(S3.T @ k, v) < 1e-12


def test_retention_equals_its_sum_over_earlier_tokens():
    g = torch.Generator().manual_seed(6)
    T, D, H, d, dv = 10, 8, 2, 4, 3
    m = {"heads": H, "dim": d, "vdim": dv, "decay": [0.5, 0.9], "rot": {"dims": 4, "base": 10.0}}
    w = {"x.q": torch.randn(H * d, D, generator=g, dtype=F), "x.k": torch.randn(H * d, D, generator=g, dtype=F),
         "x.v": torch.randn(H * dv, D, generator=g, dtype=F), "x.g": torch.randn(H * dv, D, generator=g, dtype=F),
         "x.o": torch.eye(H * dv, dtype=F)}
    h = torch.randn(T, D, generator=g, dtype=F)
    got = P.retention(h, w, "x.", m, 1e-6)
    pos = torch.arange(T)
    q = P.rotate((h @ w["x.q"].T).view(T, H, d), pos, m["rot"], "half")
    k = P.rotate((h @ w["x.k"].T).view(T, H, d), pos, m["rot"], "half") * d ** -0.5
    v = (h @ w["x.v"].T).view(T, H, dv)
    o = torch.zeros(T, H, dv, dtype=F)
    for t in range(T):
        for s in range(t + 1):
            for head in range(H):
                o[t, head] += m["decay"][head] ** (t - s) * float(q[t, head] @ k[s, head]) * v[s, head]
    want = P.unit_rms(o, 1e-6).reshape(T, -1) * P.silu(h @ w["x.g"].T)
    assert util.rel_err(got, want) < 1e-12


def test_the_router_by_hand():
    s = torch.tensor([[0.60, 0.50, 0.90, 0.05, 0.55, 0.45]], dtype=F)
    z = torch.log(s / (1 - s))
    corr = torch.tensor([0.0, 0.0, 0.0, 0.0, 0.1, 0.0], dtype=F)
    # groups of two: 1.10, 0.95, 1.10 with the correction; groups 0 and 2 stay; experts 4 (0.65)
    # and 0 (0.60) are chosen; their weights come from s, 0.55 and 0.60
    chosen, weights = P.route(z, corr, 2, 3, 2)
    assert chosen.tolist() == [[4, 0]]
    assert util.rel_err(weights, torch.tensor([[0.55 / 1.15, 0.60 / 1.15]], dtype=F)) < 1e-12
    # all choice scores negative: the kept group's experts still win over the others
    chosen, _ = P.route(z, torch.tensor([-5.0, -5.0, -9.0, -9.0, -9.0, -9.0], dtype=F), 2, 3, 1)
    assert sorted(chosen.tolist()[0]) == [0, 1]
    # groups of one expert: a group's score is that expert's
    chosen, _ = P.route(z, torch.zeros(6, dtype=F), 2, 6, 3)
    assert sorted(chosen.tolist()[0]) == [0, 2]


def test_which_matrix_is_the_gate_and_the_shared_expert_s_factor():
    g = torch.Generator().manual_seed(7)
    D, Fi = 6, 4
    h = torch.randn(3, D, generator=g, dtype=F).abs() + 0.1
    gate, up, down = (torch.randn(Fi, D, generator=g, dtype=F), torch.randn(Fi, D, generator=g, dtype=F),
                      torch.randn(D, Fi, generator=g, dtype=F))
    # a large negative pre-activation of the gate silences the expert; of the up matrix it does not
    assert float(P.gated_expert(h, gate * 0 - 50.0, up, down).abs().max()) < 1e-9
    assert float(P.gated_expert(h, gate, up * 0 - 50.0, down).abs().max()) > 1e-3


# --------------------------------------------------------------------------- configuration and layout
def test_the_configuration_reader_and_what_it_refuses():
    import gpt_fast_amd as gfa
    from gpt_fast_amd.config.refolix import ConfigError, RefolixConfig
    for name, config in CASES.items():
        c = RefolixConfig.from_dict(config)
        again = RefolixConfig.from_dict(c.to_dict())
        assert again == c, name
        arch = gfa.config.registry.architecture_of(config)
        plan = arch.plan(c)
        assert len(plan.layers) == len(config["layers"])
    c = RefolixConfig.from_dict(CASES["A"])
    left = c.layers[0].mixer.left
    assert (left.heads, left.kv_heads, left.dim, left.vdim, left.window, left.softcap) == (6, 3, 24, 16, 40, 15.0)
    assert left.rot.scaling == (4.0, 64.0, 16.0, 2.0) and c.layers[2].mlp is None
    assert c.alpha == 2.0 and c.embedding_scale == 1.5 and c.logit_scale == 0.5 and c.logit_softcap == 20.0

    def broken(change):
        config = copy.deepcopy(CASES["A"])
        change(config)
        with pytest.raises(ConfigError):
            RefolixConfig.from_dict(config)
    broken(lambda c: c["layers"][0].update(type="other"))
    broken(lambda c: c["layers"][0]["mixer"]["left"].update(kv_heads=4))
    broken(lambda c: c["layers"][0]["mixer"]["right"].update(kv_heads=3))
    broken(lambda c: c["layers"][0]["mixer"]["left"]["rot"].update(dims=7))
    broken(lambda c: c["layers"][0]["mixer"]["left"]["rot"].update(dims=26))
    broken(lambda c: c["layers"][1]["mixer"].update(decay=[0.5]))
    broken(lambda c: c["layers"][0]["mlp"]["router"].update(top=5))
    broken(lambda c: c["layers"][0]["mlp"]["router"]["groups"].update(count=4))
    broken(lambda c: c.pop("vocab"))
    broken(lambda c: c["layers"][0]["mixer"]["right"].pop("conv"))


@pytest.mark.parametrize("name", sorted(CASES))
def test_the_layout_names_every_parameter_of_the_model(tmp_path, name):
    import gpt_fast_amd as gfa
    from gpt_fast_amd.parts.base import Runtime
    from gpt_fast_amd.parts.model import DecoderModel
    from gpt_fast_amd.weights.bindings import load_parameters
    arch = gfa.config.registry.architecture_of(CASES[name])
    c = arch.read_config(CASES[name])
    model = DecoderModel(arch.plan(c), Runtime(torch.float32, "cpu"))
    declared = model.parameters()
    layout = arch.bindings(c)
    assert {b.target for b in layout.bindings} == set(declared)
    folder = make_folder(tmp_path, name, seed=1)
    params = load_parameters(folder, arch.layouts(c), "float32", None)
    for target, p in declared.items():
        assert tuple(params[target].shape) == tuple(p.shape), target
    # an expert's gate rows stand before its up rows, the experts one after the other
    _, w = P.load_folder(folder)
    for i, layer in enumerate(CASES[name]["layers"]):
        if layer["mlp"] is not None:
            ff = layer["mlp"]["expert"]["ff"]
            up = params[f"l{i}.mlp.w_up"].double()
            assert torch.equal(up[1, :ff], w[f"l{i}.mlp.e1.gate"]) and torch.equal(up[1, ff:], w[f"l{i}.mlp.e1.up"])
    assert "decayed_memory" in model.kernel_libraries() or "gated_delta" in model.kernel_libraries()


def test_a_folder_that_lacks_a_tensor_is_refused_with_its_name(tmp_path):
    import os

    import gpt_fast_amd as gfa
    from gpt_fast_amd.weights.bindings import WeightsError, load_parameters
    from gpt_fast_amd.weights.safetensors_io import write_safetensors
    from plain_llama import read_safetensors
    folder = make_folder(tmp_path, "O", seed=2, dtype="float32")
    path = os.path.join(folder, "model.safetensors")
    tensors = read_safetensors(path)
    del tensors["l0.mlp.correction"]
    tensors["l0.mix.left.q.norm"] = tensors["l0.mix.left.q.norm"][:-1].clone()
    write_safetensors(path, tensors)
    arch, c = gfa.read_model_folder(folder)
    with pytest.raises(WeightsError) as e:
        load_parameters(folder, arch.layouts(c), "float32", None)
    assert "l0.mlp.correction" in str(e.value) and "l0.mix.left.q.norm" in str(e.value)


def test_random_cases_are_read_and_run_by_the_plain_implementation(tmp_path):
    import os

    from gpt_fast_amd.config.refolix import RefolixConfig
    from refolix_cases import write_model
    for seed in (1, 2):
        config = random_case(seed)
        RefolixConfig.from_dict(config)
        folder = write_model(os.path.join(str(tmp_path), f"r{seed}"), config, seed)
        cfg, w = P.load_folder(folder)
        toks = util.random_tokens(cfg["vocab"], 30, seed)
        outs = []
        logits = P.forward(w, cfg, toks, outs)
        assert logits.shape == (30, cfg["vocab"]) and torch.isfinite(logits).all() and len(outs) == len(cfg["layers"])
        # causal: the logits of a prefix are the prefix of the logits
        assert util.rel_err(P.forward(w, cfg, toks[:11]), logits[:11]) < 1e-9


# --------------------------------------------------------------------------- the joint cache need
def test_a_joint_need_keeps_pages_and_state_side_by_side():
    from gpt_fast_amd.cache.slots import CacheFull
    from gpt_fast_amd.cache.store import Cache, JointNeed, KVNeed, StateNeed
    joint = JointNeed((KVNeed(2, 8, 70, 4), StateNeed((5,), "float32")))
    needs = [joint, StateNeed((3,), "float32"), joint, None]
    cache = Cache(needs, [None] * 4, max_tokens=64 * 5, max_sequences=3, dtype=torch.float32, device="cpu")
    assert len(cache.groups) == 2 and cache.entries[3] is None
    e0, e2 = cache.entries[0], cache.entries[2]
    assert e0.group is e2.group and (e0.index, e2.index) == (0, 1)
    kv, st = e0.part(0), e0.part(1)
    assert kv.k_pages.shape[1:] == (2, 64, 8) and kv.v_pages.shape[1:] == (2, 4, 64) and st.state.shape == (4, 5)
    assert kv.group_id == e0.group_id and [gid for gid, _ in cache.paged_groups] == [e0.group_id]
    a = cache.acquire()
    st.state[a].fill_(3.0)
    cache.extend(a, 130)
    assert len(cache.page_list(e0.group_id, a)) == 3
    cache.extend(a, 70)
    cache.extend(a, 1)                       # from 200 tokens on, a window of 70 needs no key before 131
    held = cache.page_list(e0.group_id, a)
    assert held[:2] == [-1, -1] and len(held) == 4 and sum(p >= 0 for p in held) == 2
    row = torch.zeros(6, dtype=torch.int32).numpy()
    e0.group.fill_table_row(row, a)
    assert list(row[:4]) == held and list(row[4:]) == [-1, -1]
    b = cache.acquire()
    with pytest.raises(CacheFull):
        cache.extend(b, 64 * 4)              # three pages are free
    cache.check()
    cache.release(a)
    c = cache.acquire()
    assert c == a and float(e0.part(1).state[c].abs().max()) == 0.0       # a slot that comes back starts clean
    cache.extend(b, 64 * 3)
    cache.check()
    cache.release(b)
    cache.release(c)
    assert e0.group.pages.held == 0
    with pytest.raises(ValueError):
        Cache([JointNeed((KVNeed(1, 8), KVNeed(1, 8)))], [None], max_tokens=64, max_sequences=1,
              dtype=torch.float32, device="cpu")
